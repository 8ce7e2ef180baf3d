"""Writes tests/golden/vectors.npz: small input/expected-output vectors for the hot path.

The reference repository holds no fixture files for gather / scatter-accumulate (its only
known-answer vector, the ``i + 2r`` pattern of examples/all_gather.py:80-84,121-125, is a closed
form and is generated inside the tests). These vectors are therefore produced by THIS repository's
CPU oracle (oracle/odc_oracle.py), after the oracle itself has been pinned by tests/test_oracle.py.
They serve two purposes: the oracle cannot drift unnoticed, and the GPU tests can check the HIP path
against committed data as well as against the live oracle.

Inputs are built with integer arithmetic only (a multiplicative hash of the index), so the file is
reproducible on any machine:  python tests/golden/make_vectors.py
"""

import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parent.parent.parent
sys.path.insert(0, str(ROOT))

from oracle import odc_oracle as oracle  # noqa: E402

OUT = Path(__file__).resolve().parent / "vectors.npz"


def hashed_bits16(n: int, salt: int) -> torch.Tensor:
    """n pseudo-random 16-bit patterns; exponent all-ones (Inf/NaN) is avoided."""
    i = torch.arange(n, dtype=torch.int64)
    h = ((i + salt) * 2654435761 + 0x9E3779B9 * salt) & 0xFFFFFFFF
    h = (h ^ (h >> 15)) * 2246822519 & 0xFFFFFFFF
    return ((h >> 13) & 0xFFFF).to(torch.int32)


def bf16_values(n, salt):
    b = hashed_bits16(n, salt)
    b = torch.where((b & 0x7F80) == 0x7F80, b & ~0x4000, b)  # keep finite
    b = (b & 0x8000) | ((((b >> 7) & 0xFF) % 40 + 100) << 7) | (b & 0x7F)  # exponents 100..139: ~1e-8..1e3
    return b.to(torch.int16).view(torch.bfloat16)


def fp16_values(n, salt):
    b = hashed_bits16(n, salt)
    b = (b & 0x8000) | ((((b >> 10) & 0x1F) % 20 + 5) << 10) | (b & 0x3FF)
    return b.to(torch.int16).view(torch.float16)


def bits(t):
    return t.contiguous().view({2: torch.int16, 4: torch.int32}[t.element_size()]).numpy()


def main():
    v = {}
    # gather, W=3, odd shard size
    W, S = 3, 37
    shards = [hashed_bits16(S, 10 + r).to(torch.int16) for r in range(W)]
    v["gather_shards"] = np.stack([s.numpy() for s in shards])
    v["gather_out"] = oracle.gather(shards).numpy()
    # scatter-accumulate, three microbatches, three dtype pairs, shard size not a multiple of 4
    W, S, M = 4, 1001, 3
    for tag, make, acc_dtype in (("bf16_f32", bf16_values, torch.float32), ("f16_f32", fp16_values, torch.float32),
                                 ("bf16_bf16", bf16_values, torch.bfloat16)):
        grads = [make(W * S, 100 + m) for m in range(M)]
        accs = [torch.zeros(S, dtype=acc_dtype) for _ in range(W)]
        for g in grads:
            oracle.scatter_accumulate(accs, g)
        v[f"acc_{tag}_grads"] = np.stack([bits(g) for g in grads])
        v[f"acc_{tag}_out"] = np.stack([bits(a) for a in accs])
    # FSDP1 flat parameter: numel not divisible by W, padded shards and padded gradient
    W, n = 4, 1003
    flat = bf16_values(n, 7)
    v["fsdp1_flat"] = bits(flat)
    v["fsdp1_shards"] = np.stack([bits(oracle.fsdp1_get_shard(flat, r, W)) for r in range(W)])
    accs = [torch.zeros(-(-n // W)) for _ in range(W)]
    grad = bf16_values(n, 8)
    oracle.scatter_accumulate(accs, oracle.fsdp1_pad_grad(grad, W))
    v["fsdp1_grad"] = bits(grad)
    v["fsdp1_acc"] = np.stack([bits(a) for a in accs])
    v["fsdp1_published_div4_bf16"] = bits(oracle.fsdp1_publish(accs[1].clone(), 4.0, torch.bfloat16))
    # a divisor that is not a power of two: the quotient must be the correctly rounded one
    v["fsdp2_averaged_div12"] = bits(oracle.fsdp2_average(accs[2].clone(), 12))
    # gather with cast fp32 -> bf16
    W, S = 4, 259
    f32 = [bf16_values(S, 50 + r).float() * 1.00390625 for r in range(W)]  # off the bf16 grid: rounding happens
    v["cast_shards"] = np.stack([bits(s) for s in f32])
    v["cast_out"] = bits(oracle.gather_cast(f32, torch.bfloat16))
    np.savez_compressed(OUT, **v)
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes, {len(v)} arrays)")


if __name__ == "__main__":
    main()
