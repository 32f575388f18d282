"""Writes the small input/output vectors under tests/golden/.

These fixtures are SELF-GENERATED from this repository's CPU oracle
(oracle/attention_oracle.py, fp64): the reference repository holds no golden
vectors, known-answer tests or stored fixtures for this path (its tests draw
CUDA random numbers at run time), and its own implementation cannot run without
flash-attn.  The vectors freeze the oracle (a later edit that changes its
results fails tests/test_golden.py on CPU) and give the GPU tests a second,
file-based target.  Inputs are bf16-representable so the kernels see exactly
the same numbers.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import attention_oracle as O  # noqa: E402


def bf16_grid(*shape, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).bfloat16().double()


def save(name, **arrays):
    out = {k: (v.numpy() if torch.is_tensor(v) else np.asarray(v)) for k, v in arrays.items()}
    out = {k: (a.astype(np.float32) if a.dtype == np.float64 else a) for k, a in out.items()}
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **out)


def main():
    # 1. dense sliding window, GQA 2:1, head_dim 64, window 10
    q, k, v, do = bf16_grid(1, 40, 4, 64, seed=1), bf16_grid(1, 40, 2, 64, seed=2), \
        bf16_grid(1, 40, 2, 64, seed=3), bf16_grid(1, 40, 4, 64, seed=4)
    out, lse, dq, dk, dv = O.attention_fwd_bwd(
        lambda q, k, v: O.sliding_window_attn(q, k, v, 10, compute_dtype=torch.float64), q, k, v, do)
    save("swa_dense", q=q, k=k, v=v, do=do, window=np.int32(10), out=out, lse=lse, dq=dq, dk=dk, dv=dv)

    # 2. streaming-LLM, one sink, window 6
    out, lse, dq, dk, dv = O.attention_fwd_bwd(
        lambda q, k, v: O.streaming_llm_attn(q, k, v, 6, n_sink=1, compute_dtype=torch.float64),
        q, k, v, do)
    save("slm_dense", q=q, k=k, v=v, do=do, window=np.int32(6), n_sink=np.int32(1),
         out=out, lse=lse, dq=dq, dk=dk, dv=dv)

    # 3. packed sliding window, lengths 7 / 21 / 12, window 5
    cu = np.array([0, 7, 28, 40], dtype=np.int32)
    qp, kp, vp, dop = q[0], k[0], v[0], do[0]
    out, lse, dq, dk, dv = O.attention_fwd_bwd(
        lambda q, k, v: O.sliding_window_attn_varlen(q, k, v, 5, cu, compute_dtype=torch.float64),
        qp, kp, vp, dop)
    save("swa_varlen", q=qp, k=kp, v=vp, do=dop, cu_seqlens=cu, window=np.int32(5),
         out=out, lse=lse, dq=dq, dk=dk, dv=dv)

    # 4. LSE merge with the ring's dtypes (fp32 o / fp64 lse / bf16 new o / fp32 new lse)
    g = torch.Generator().manual_seed(5)
    o = torch.randn(1, 24, 2, 64, generator=g).float()
    l = (3 * torch.randn(1, 2, 24, generator=g)).double()
    on = torch.randn(1, 24, 2, 64, generator=g).bfloat16()
    ln = (3 * torch.randn(1, 2, 24, generator=g)).float()
    l[0, 0, 3] = float("-inf")
    ln[0, 1, 5] = float("-inf")
    om, lm = O.merge(o.double(), l, on.double(), ln.double())
    save("merge_ring", o=o, lse=l, o_new=on.float(), lse_new=ln, o_merged=om, lse_merged=lm)


if __name__ == "__main__":
    main()
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
