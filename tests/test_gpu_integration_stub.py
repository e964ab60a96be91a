"""The ctypes binding a maintainer of the reference would add at its patch point
(utils/rs_overlap.py:438-441), executed as it is written: the first Python code block under the
"Seam 2" heading of the integration guide at the repository root is extracted, run against the built
library, and its two functions are compared with the CPU oracle on a small layer whose sizes are
multiples of 64."""
import os
import re

import pytest
import torch

from oracle import ref_moe
from sparse_amd import _lib
from tests.helpers import make_hidden, make_layer

pytestmark = pytest.mark.gpu

_DOC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "INTEGRATION.md")


def _stub_source() -> str:
    text = open(_DOC).read()
    seam = text.index("## Seam 2")
    m = re.search(r"```python\n(.*?)```", text[seam:], re.S)
    assert m, "no Python block under Seam 2"
    return m.group(1)


@pytest.fixture(scope="module")
def stub():
    _lib.load()                                   # fails loudly if the library is not built
    os.environ["SPARSE_HIP_LIB"] = str(_lib.LIB_PATH)
    ns = {}
    exec(compile(_stub_source(), "INTEGRATION.md:seam-2", "exec"), ns)
    return ns


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T", [8, 96])
@pytest.mark.parametrize("renorm", [False, True])
def test_stub_matches_oracle(stub, device, dtype, T, renorm):
    H, E, I, K = 128, 8, 64, 2
    layer = make_layer(H, E, I, K, dtype=dtype, seed=3, std=0.05)
    x = make_hidden(T, H, dtype, seed=4 + T)
    want_v, want_i, want_logits = ref_moe.routing_router(x, layer["gate_w"], K, renorm)
    xd = x.to(device)
    topv, topi, logits = stub["routing_router"](xd, layer["gate_w"].to(device), K, renorm)
    # the gate: fp32 accumulation rounded once on the device, library GEMM on the host: last-bit differences
    torch.testing.assert_close(logits.cpu().float(), want_logits.float(), rtol=2e-2, atol=2e-2)
    # indices and weights are exact given identical logits
    v2, i2, _ = ref_moe.routing_router(x, layer["gate_w"], K, renorm, router_logits=logits.cpu())
    assert torch.equal(topi.cpu(), i2)
    torch.testing.assert_close(topv.cpu().float(), v2.float(), rtol=2 ** -7 if dtype == torch.bfloat16 else 2 ** -10,
                               atol=0)
    slab, slot = stub["load_experts"]([tuple(w.to(device) for w in ex) for ex in layer["experts"]])
    out = stub["experts_world1_exact"](slab, slot, xd, topv, topi, E, H, I)
    want = ref_moe.experts_world1_exact(x, topi.cpu(), topv.cpu(), layer["experts"])
    # 16-bit outputs of fp32-accumulated products of different summation order: two roundings apart at most
    tol = 2 ** -6 if dtype == torch.bfloat16 else 2 ** -9
    torch.testing.assert_close(out.cpu().float(), want.float(), rtol=tol, atol=tol * float(want.float().abs().max()))


def test_stub_fp32(stub, device):
    H, E, I, K, T = 64, 4, 64, 2, 5
    layer = make_layer(H, E, I, K, dtype=torch.float32, seed=5, std=0.05)
    x = make_hidden(T, H, torch.float32, seed=6)
    topv, topi, _ = stub["routing_router"](x.to(device), layer["gate_w"].to(device), K, True)
    slab, slot = stub["load_experts"]([tuple(w.to(device) for w in ex) for ex in layer["experts"]])
    from sparse_amd.weights import tile_weight
    assert torch.equal(slab[1, :I * H].cpu(), tile_weight(layer["experts"][1][0]))
    out = stub["experts_world1_exact"](slab, slot, x.to(device), topv, topi, E, H, I)
    want = ref_moe.experts_world1_exact(x, topi.cpu(), topv.cpu(), layer["experts"])
    torch.testing.assert_close(out.cpu(), want, rtol=1e-4, atol=1e-6)


def test_stub_reports_errors_like_the_binding_says(stub, device):
    x = torch.zeros((4, 60), device=device, dtype=torch.bfloat16)          # H % 8 != 0
    with pytest.raises(ValueError):
        stub["routing_router"](x, torch.zeros((8, 60), device=device, dtype=torch.bfloat16), 2, False)
