"""The dK/dV kernel issues its S and dP MFMAs as inline assembly (accumulators in vector
registers) and keeps the distance between such an MFMA and the first read of its result by
hand: the compiler does not know these statements are MFMAs and pads nothing.  The build also
produces the library with every MFMA issued through the compiler builtin, where the compiler
pads each hazard itself.  Both run the same arithmetic in the same order, so their outputs must
agree bit for bit; a result read too early in the hand-scheduled build would differ."""
import os

import pytest
import torch

pytestmark = pytest.mark.gpu

CASES = [
    dict(b=1, sq=2048, sk=2048, hq=8, hk=2, d=128, window=(512, 0), causal=True, sink=0),
    dict(b=2, sq=777, sk=901, hq=4, hk=4, d=64, window=(-1, -1), causal=True, sink=0),
    dict(b=1, sq=1500, sk=1500, hq=4, hk=1, d=128, window=(200, 0), causal=True, sink=3),
    dict(b=1, sq=640, sk=512, hq=2, hk=2, d=64, window=(40, 90), causal=False, sink=0),
    dict(b=1, sq=4096, sk=4096, hq=4, hk=1, d=128, window=(0, 8192), causal=False, sink=0),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("case", CASES, ids=[f"case{i}" for i in range(len(CASES))])
def test_inline_asm_and_builtin_mfma_builds_agree_bit_for_bit(case, dtype, monkeypatch):
    from ring_swa import _lib
    from ring_swa.ops import attn_bwd, attn_fwd

    alt_path = os.path.join(os.path.dirname(_lib.LIB_PATH), "librswa_builtin_mfma.so")
    assert os.path.exists(alt_path), f"{alt_path} is missing: run build.py"
    torch.manual_seed(3)
    b, d = case["b"], case["d"]
    mk = lambda s, h: torch.randn(b, s, h, d, device="cuda").to(dtype)  # noqa: E731
    q, do = mk(case["sq"], case["hq"]), mk(case["sq"], case["hq"])
    k, v = mk(case["sk"], case["hk"]), mk(case["sk"], case["hk"])
    out, lse = attn_fwd(q, k, v, None, case["window"], case["causal"], num_sink=case["sink"])

    def backward():
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        attn_bwd(q, k, v, out, lse, do, dq, dk, dv, None, case["window"], case["causal"],
                 num_sink=case["sink"])
        return dq, dk, dv

    main = backward()
    _lib.lib()
    monkeypatch.setattr(_lib, "_lib", _lib.load(alt_path))
    alt = backward()
    for name, x, y in zip(("dq", "dk", "dv"), main, alt):
        assert torch.isfinite(x.float()).all()
        assert torch.equal(x, y), name
