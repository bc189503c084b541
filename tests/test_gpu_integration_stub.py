"""The binding that the integration guide at the repository root proposes for the reference (its option B), executed
verbatim: the stub text is cut out of the document, exec'd, and called exactly as boilerplate/kernels/ternary_cuda.py:98-103 calls its native module
(11 positional arguments, float32 scales from `w_scale.float()`, a real `lut1` tensor, device offsets)."""

import re
from pathlib import Path

import numpy as np
import pytest
import torch

from _util import c_gemm, orc, rel_l2, synth_weights

pytestmark = pytest.mark.gpu

ROOT = Path(__file__).resolve().parent.parent


def _stub_class():
    text = (ROOT / "INTEGRATION.md").read_text()
    blocks = re.findall(r"```python\n(.*?)```", text, flags=re.S)
    code = next(b for b in blocks if "class _Hip" in b)
    ns = {}
    exec(compile(code, "INTEGRATION.md:option-B", "exec"), ns)
    return ns["_Hip"]


@pytest.mark.parametrize("fmt,K,counts", [("tq2", 2048, [3, 0, 5]), ("tq1", 2048, [1, 1, 1]), ("tq1", 4096, [20, 3, 9]), ("tq2", 200, [2, 1, 4])])
def test_option_b_stub_runs_the_reference_call(fmt, K, counts):
    from deepseekternarized_amd.kernels import _lib

    hip = _stub_class()(str(_lib.LIB_PATH))
    E, N, group = len(counts), 48, 64 if K == 200 else 128
    rng = np.random.default_rng(K)
    packed, scales = synth_weights(K, E, N, K, group, fmt)
    offs = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
    T = int(offs[-1])
    q, s = orc.quant_act_int8(rng.standard_normal((T, K)).astype(np.float32))
    dev = torch.device("cuda")
    # boilerplate/kernels/ternary_cuda.py:94-103, line for line
    x, x_scale = torch.from_numpy(q).to(dev), torch.from_numpy(s).to(dev)
    packed_t, w_scale = torch.from_numpy(packed[0]).to(dev), torch.from_numpy(scales[0]).to(dev)
    lut1 = torch.from_numpy(orc.tq1_lut()).to(dev)
    offs_t = torch.from_numpy(offs)
    max_rows = int(offs_t.diff().max())
    out = torch.zeros(x.size(0), packed_t.size(1), dtype=torch.float32, device=dev)
    hip.ternary_grouped_gemm(out, x.contiguous(), x_scale.float().contiguous(), offs_t.to(dev), packed_t.contiguous(),
                             w_scale.float().contiguous(), K, group, 2 if fmt == "tq2" else 1, lut1, max_rows)
    want = np.zeros((T, N), np.float32)
    for e in range(E):
        a, b = int(offs[e]), int(offs[e + 1])
        if b > a:
            c_gemm(q[a:b], s[a:b], packed[0][e], scales[0][e].astype(np.float32), K, group, fmt, out=want[a:b])
    got = out.cpu().numpy()
    assert rel_l2(got, want) <= 1e-3
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-3)  # the reference's own tolerance (tests/test_ternary_cuda.py:80,87)


def test_option_b_stub_raises_runtime_error_with_the_library_message():
    from deepseekternarized_amd.kernels import _lib

    hip = _stub_class()(str(_lib.LIB_PATH))
    dev = torch.device("cuda")
    out = torch.zeros(2, 16, device=dev)
    x = torch.zeros(2, 256, dtype=torch.int8, device=dev)
    xs = torch.ones(2, device=dev)
    packed = torch.zeros(1, 16, 63, dtype=torch.uint8, device=dev)  # 63 != ceil(256 / 4)
    ws = torch.ones(1, 16, 2, device=dev)
    with pytest.raises(RuntimeError, match="inconsistent"):
        hip.ternary_grouped_gemm(out, x, xs, torch.tensor([0, 2], device=dev), packed, ws, 256, 128, 2, torch.zeros(256, 5, dtype=torch.int8, device=dev), 2)
