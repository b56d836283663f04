"""The ctypes stub that the repository's integration notes print (the stand-in for the reference's pybind pair
cal_max_coffs + self_attn_forward) is executed as written and checked against the oracle."""
import os
import re

import numpy as np
import pytest
import torch

from helpers import make_attn_case, to_half_and_back

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _stub_source():
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    blocks = re.findall(r"```python\n(.*?)```", text, flags=re.S)
    blocks = [b for b in blocks if "def self_attn_forward" in b]
    assert len(blocks) == 1
    return blocks[0]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_integration_stub_runs_as_written(oracle_lib, hip_lib, dtype, monkeypatch):
    monkeypatch.chdir(ROOT)                       # the stub opens the library by its path in the source tree
    scope = {}
    exec(compile(_stub_source(), "INTEGRATION.md", "exec"), scope)
    case = make_attn_case(oracle_lib, seed=71, n=1500, ws=5, quant=4, heads=6, dim=8, extent=(9, 9, 4), batches=2,
                          recipe="layer")
    if dtype == torch.float16:
        to_half_and_back(case)
    ref, rmax, rsum, _ = oracle_lib.attn_fwd(*case.oracle_args(), return_stats=True)
    dev = torch.device("cuda")
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    f = lambda a: t(a).to(dtype)
    i = case.index
    indices = [None, t(i["w_sizes"]), None, t(i["w2n"]), t(i["n2n"]), t(case.n_coords)]
    raw, sm, mx = scope["self_attn_forward"]([f(case.q), f(case.k), f(case.v)], [f(case.tq), f(case.tk), f(case.tv)],
                                             [int(x) for x in case.table_sizes], indices)
    torch.cuda.synchronize()
    assert raw.shape == case.q.shape and sm.shape == mx.shape == (case.N, case.H, 1)
    tol = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-3, atol=2e-3)
    np.testing.assert_allclose(mx[..., 0].double().cpu().numpy(), rmax, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(sm[..., 0].double().cpu().numpy(), rsum, rtol=2e-5)
    # the reference divides raw by the sum (attn_coff.py:184); raw = normalised output times the sum
    np.testing.assert_allclose((raw.double() / sm.double()).cpu().numpy(), ref, **tol)
