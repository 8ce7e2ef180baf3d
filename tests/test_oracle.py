"""Pins the CPU oracle (oracle/odc_oracle.py) WITHOUT the HIP path: against the reference's own
known-answer pattern, closed forms, brute-force loops on tiny inputs, and an independent scalar C
restatement (oracle/odc_oracle.c). A plausible mistake in the oracle (wrong chunk index, dropped
padding, store-instead-of-add, wrong widening) fails at least one of these."""

import ctypes
import math
import subprocess
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import odc_oracle as oracle

ORACLE_DIR = Path(oracle.__file__).resolve().parent


@pytest.fixture(scope="module")
def c_oracle():
    lib_path = ORACLE_DIR / "libodc_oracle.so"
    subprocess.run(["make", "-C", str(ORACLE_DIR)], check=True, capture_output=True)
    lib = ctypes.CDLL(str(lib_path))
    lib.oracle_gather.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p), ctypes.c_uint32, ctypes.c_uint64]
    lib.oracle_scatter_accumulate_f32.argtypes = [
        ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p, ctypes.c_int, ctypes.c_uint64, ctypes.c_uint32, ctypes.c_uint64]
    lib.oracle_scatter_accumulate_bf16.argtypes = [
        ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p, ctypes.c_uint64, ctypes.c_uint32, ctypes.c_uint64]
    lib.oracle_widen_bf16.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64]
    lib.oracle_widen_f16.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64]
    lib.oracle_narrow_bf16.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64]
    lib.oracle_divide_f32.argtypes = [ctypes.c_void_p, ctypes.c_float, ctypes.c_uint64]
    return lib


def _ptrs(tensors):
    arr = (ctypes.c_void_p * len(tensors))()
    for i, t in enumerate(tensors):
        arr[i] = t.data_ptr()
    return arr


def _bits(t):
    return t.contiguous().view({2: torch.int16, 4: torch.int32, 8: torch.int64}[t.element_size()])


GRAD_KIND = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}


# ---- gather ------------------------------------------------------------------------------------
def test_gather_reference_known_answer():
    """examples/all_gather.py:80-84,121-125: tensor i of rank r holds i + 2r (int64); block r of the
    gathered tensor equals 2r + i."""
    W, size = 8, 1024
    for i in range(20):
        shards = [torch.full((size,), i + 2 * r, dtype=torch.int64) for r in range(W)]
        for local_rank in (0, 3, W - 1):
            dst = torch.empty(size * W, dtype=torch.int64)
            oracle.gather_into_tensor(dst, shards, local_rank)
            for r in range(W):
                assert torch.eq(dst[r * size : (r + 1) * size], 2 * r + i).all()
        assert torch.equal(oracle.gather(shards), dst)


@pytest.mark.parametrize("W", [1, 2, 3, 5, 8, 12, 64])
@pytest.mark.parametrize("S", [0, 1, 63, 64, 65, 257])
def test_gather_brute_force(W, S, c_oracle):
    g = torch.Generator().manual_seed(W * 31 + S)
    shards = [torch.randint(-(2**15), 2**15 - 1, (S,), generator=g, dtype=torch.int16) for _ in range(W)]
    out = torch.full((W * S + 8,), -999, dtype=torch.int16)
    oracle.gather_into_tensor(out[4 : 4 + W * S], shards, local_rank=W // 2)
    for r in range(W):
        for j in range(S):
            assert out[4 + r * S + j].item() == shards[r][j].item()
    assert (out[:4] == -999).all() and (out[4 + W * S :] == -999).all()  # sentinel, tests/nvshmem_triton/test_getmem.py:93-112
    if S:
        c_out = torch.empty(W * S, dtype=torch.int16)
        c_oracle.oracle_gather(c_out.data_ptr(), _ptrs(shards), W, S * 2)
        assert torch.equal(c_out, out[4 : 4 + W * S])


def test_gather_is_a_byte_copy_for_every_bf16_pattern():
    allbits = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    shards = list(allbits.view(4, -1))
    assert torch.equal(_bits(oracle.gather(shards)), _bits(allbits))


def test_gather_cast_rounds_to_nearest_even(c_oracle):
    g = torch.Generator().manual_seed(17)
    vals = torch.cat([
        torch.randn(100_000, generator=g),
        torch.randn(10_000, generator=g) * 1e-30, torch.randn(10_000, generator=g) * 1e30,
        torch.tensor([1.0 + 2.0**-8, 1.0078125 + 2.0**-8, -(1.0 + 2.0**-8), 3.3895e38, 3.4e38, 1e-45, -0.0, 0.0,
                      float("inf"), -float("inf")]),
        (2.0 ** torch.arange(-149, 128, dtype=torch.float64)).float() * 1.00390625,  # ties at every exponent
    ])
    vals = torch.cat([vals, torch.zeros((-vals.numel()) % 4)])
    shards = list(vals.view(4, -1))
    got = oracle.gather_cast(shards, torch.bfloat16)
    want = torch.empty(vals.numel(), dtype=torch.int16)
    c_oracle.oracle_narrow_bf16(want.data_ptr(), vals.data_ptr(), vals.numel())
    assert torch.equal(_bits(got), want)
    assert got[100_000 + 20_000].item() == 1.0 and got[100_000 + 20_001].item() == 1.015625  # ties to even
    # widening is exact
    b = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    wide = oracle.gather_cast(list(b.view(8, -1)), torch.float32)
    ok = ~torch.isnan(wide)
    assert torch.equal(_bits(wide[ok]), (b.view(torch.int16).to(torch.int32) << 16)[ok])


def test_division_matches_numpy_float32():
    g = torch.Generator().manual_seed(19)
    acc = torch.randn(50_000, generator=g) * 1e-2
    for W in (1, 2, 3, 7, 8, 12, 64):
        want = torch.from_numpy(acc.numpy() / np.float32(W))
        assert torch.equal(_bits(oracle.fsdp2_average(acc.clone(), W)), _bits(want))
        got = oracle.fsdp1_publish(acc.clone(), float(W), torch.bfloat16)
        assert torch.equal(_bits(got), _bits(want.bfloat16() if W > 1 else acc.bfloat16()))


# ---- scatter-accumulate ------------------------------------------------------------------------
def test_scatter_accumulate_closed_forms():
    W, S, M = 4, 1000, 37
    accs = [torch.zeros(S) for _ in range(W)]
    for _ in range(M):
        oracle.scatter_accumulate(accs, torch.ones(W * S, dtype=torch.bfloat16))
    assert all((a == M).all() for a in accs)  # ones x M == M exactly
    accs = [torch.zeros(S) for _ in range(W)]
    for k in range(-20, 21):
        oracle.scatter_accumulate(accs, torch.full((W * S,), 2.0**k, dtype=torch.bfloat16))
    assert all((a == sum(2.0**k for k in range(-20, 21))).all() for a in accs)  # exact in fp32
    # chunk r of the gradient goes to rank r, element for element
    grad = torch.arange(W * S, dtype=torch.float32)
    accs = [torch.zeros(S) for _ in range(W)]
    oracle.scatter_accumulate(accs, grad)
    for r in range(W):
        assert torch.equal(accs[r], torch.arange(r * S, (r + 1) * S, dtype=torch.float32))


def test_scatter_accumulate_signed_zero_and_specials():
    W = 2
    accs = [torch.zeros(4) for _ in range(W)]
    oracle.scatter_accumulate(accs, torch.full((8,), -0.0, dtype=torch.bfloat16))
    assert not any(torch.signbit(a).any() for a in accs)  # +0 + -0 = +0: the first call must ADD
    accs = [torch.full((4,), -0.0) for _ in range(W)]
    oracle.scatter_accumulate(accs, torch.full((8,), -0.0, dtype=torch.bfloat16))
    assert all(torch.signbit(a).all() for a in accs)  # -0 + -0 = -0
    accs = [torch.zeros(4) for _ in range(W)]
    specials = torch.tensor([float("inf"), -float("inf"), float("nan"), 3.3895e38, 1e-40, -1e-40, 1.0, -1.0]).bfloat16()
    oracle.scatter_accumulate(accs, specials)
    got = torch.cat(accs)
    assert got[0] == float("inf") and got[1] == -float("inf") and torch.isnan(got[2])
    assert torch.equal(got[3:], specials[3:].float())  # 0 + x == x exactly, bf16 denormals included
    oracle.scatter_accumulate(accs, specials)
    assert torch.isnan(torch.cat(accs)[2]) and torch.cat(accs)[0] == float("inf")


@pytest.mark.parametrize("grad_dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_scatter_accumulate_matches_c_restatement(grad_dtype, c_oracle):
    """Independent implementation: bf16 widening by a 16-bit shift, fp16 widening by field
    manipulation, one binary32 add (gcc -ffp-contract=off)."""
    W, S, M = 5, 4099, 4
    g = torch.Generator().manual_seed(3)
    accs = [torch.zeros(S) for _ in range(W)]
    c_accs = [torch.zeros(S) for _ in range(W)]
    for m in range(M):
        grad = (torch.randn(W * S, generator=g) * 10.0 ** (m - 2)).to(grad_dtype)
        oracle.scatter_accumulate(accs, grad)
        c_oracle.oracle_scatter_accumulate_f32(_ptrs(c_accs), grad.data_ptr(), GRAD_KIND[grad_dtype], W * S, W, S)
    for a, c in zip(accs, c_accs):
        assert torch.equal(_bits(a), _bits(c))


def test_widening_of_every_16_bit_pattern(c_oracle):
    allbits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    for dtype, fn in ((torch.bfloat16, c_oracle.oracle_widen_bf16), (torch.float16, c_oracle.oracle_widen_f16)):
        out = torch.empty(65536)
        fn(out.data_ptr(), allbits.data_ptr(), 65536)
        want = allbits.view(dtype).float()
        nan = torch.isnan(want)
        assert torch.equal(torch.isnan(out), nan)
        assert torch.equal(_bits(out[~nan]), _bits(want[~nan]))
        # accumulate every pattern into zero and into one: same as the C restatement
        for init in (0.0, 1.0):
            accs = [torch.full((65536 // 4,), init) for _ in range(4)]
            c_accs = [torch.full((65536 // 4,), init) for _ in range(4)]
            oracle.scatter_accumulate(accs, allbits.view(dtype))
            c_oracle.oracle_scatter_accumulate_f32(_ptrs(c_accs), allbits.data_ptr(), GRAD_KIND[dtype], 65536, 4, 65536 // 4)
            a, c = torch.cat(accs), torch.cat(c_accs)
            ok = ~torch.isnan(c)
            assert torch.equal(torch.isnan(a), ~ok) and torch.equal(_bits(a[ok]), _bits(c[ok]))


def test_bf16_accumulation_rounds_to_nearest_even(c_oracle):
    W, S = 2, 30_000
    g = torch.Generator().manual_seed(5)
    accs = [torch.randn(S, generator=g).bfloat16() for _ in range(W)]
    c_accs = [a.clone() for a in accs]
    for _ in range(3):
        grad = torch.randn(W * S, generator=g).bfloat16()
        oracle.scatter_accumulate(accs, grad)
        c_oracle.oracle_scatter_accumulate_bf16(_ptrs(c_accs), grad.data_ptr(), W * S, W, S)
    for a, c in zip(accs, c_accs):
        assert torch.equal(_bits(a), _bits(c))
    # ties: 1 + 2^-8 is halfway between two bf16 values and rounds to the even one (1.0)
    a = [torch.ones(1, dtype=torch.bfloat16)]
    oracle.scatter_accumulate(a, torch.tensor([2.0**-8]).bfloat16())
    assert a[0].item() == 1.0
    a = [torch.tensor([1.0078125]).bfloat16()]  # odd mantissa: the tie rounds up to 1.015625
    oracle.scatter_accumulate(a, torch.tensor([2.0**-8]).bfloat16())
    assert a[0].item() == 1.015625


def test_scatter_accumulate_split_size_invariance():
    """The reference walks a shard in sub-requests of local_buf_size (scatter_accumulate.py:649,
    381-391); the result must not depend on it."""
    W, S = 4, 10_007
    g = torch.Generator().manual_seed(7)
    grads = [torch.randn(W * S, generator=g).bfloat16() for _ in range(3)]
    results = []
    for split in (None, 64, 1000, 4096, S, S + 5):
        accs = [torch.zeros(S) for _ in range(W)]
        for grad in grads:
            oracle.scatter_accumulate(accs, grad, local_buf_size=split)
        results.append(torch.cat(accs))
    for r in results[1:]:
        assert torch.equal(_bits(r), _bits(results[0]))


def test_scatter_accumulate_equals_reduce_scatter_plus_add():
    """examples/reduce_scatter.py:96-105,163-172: W clients scatter-accumulating equals
    reduce_scatter(sum) followed by add_, within rtol=atol=5e-3 (exact for one client)."""
    W, S = 4, 2048
    g = torch.Generator().manual_seed(11)
    client_grads = [torch.rand(W * S, generator=g) for _ in range(W)]
    accs = [torch.zeros(S) for _ in range(W)]
    for grad in client_grads:  # clients arrive one after the other
        oracle.scatter_accumulate(accs, grad)
    reduced = torch.stack(client_grads).sum(0).view(W, S)
    for r in range(W):
        torch.testing.assert_close(accs[r], reduced[r], rtol=5e-3, atol=5e-3)
    one = [torch.zeros(S) for _ in range(W)]
    oracle.scatter_accumulate(one, client_grads[0])
    assert torch.equal(torch.cat(one), client_grads[0])


def test_order_sensitivity_is_at_the_ulp_level():
    W, S = 2, 50_000
    g = torch.Generator().manual_seed(13)
    grads = [(torch.randn(W * S, generator=g) * 1e-3).bfloat16() for _ in range(8)]
    fwd = [torch.zeros(S) for _ in range(W)]
    rev = [torch.zeros(S) for _ in range(W)]
    for grad in grads:
        oracle.scatter_accumulate(fwd, grad)
    for grad in reversed(grads):
        oracle.scatter_accumulate(rev, grad)
    a, b = torch.cat(fwd), torch.cat(rev)
    assert not torch.equal(a, b)  # order matters for bits ...
    torch.testing.assert_close(a, b, rtol=1e-6, atol=1e-9)  # ... but only at the fp32 rounding level


def test_clear_accumulations():
    accs = [torch.randn(10) for _ in range(3)]
    oracle.clear_accumulations(accs)
    assert all((_bits(a) == 0).all() for a in accs)  # +0.0, not -0.0


# ---- integer closed forms ----------------------------------------------------------------------
@pytest.mark.parametrize("shape,W,max_size,want_global,want_local", [
    ((27_264_000,), 8, 64 * 1024 * 1024, 27_264_000, 8_388_608),  # flat 8B-layer shard: 4 sub-requests
    ((7_340_032,), 8, 64 * 1024 * 1024, 7_340_032, 7_340_032),
    ((512,), 8, 64 * 1024 * 1024, 512, 512),
    ((100,), 8, 64 * 1024 * 1024, 100, 128),  # rounded up to 64 elements
    ((100,), 8, 0, 100, 128),  # splitting off
    ((1000, 3), 4, 1024, 1024, 256),
    ((218_112_000,), 8, 64 * 1024 * 1024, 67_108_864, 8_388_608),
])
def test_buffer_splitter_table(shape, W, max_size, want_global, want_local):
    sp = oracle.BufferSplitter(max_size)
    assert sp.get_global_buffer_size(shape) == want_global
    assert sp.get_local_buffer_size(shape, W) == want_local


def test_buffer_splitter_rejects_indivisible_world():
    with pytest.raises(AssertionError):  # 64 Mi % 12 != 0, utils.py:236-238
        oracle.BufferSplitter(64 * 1024 * 1024).get_local_buffer_size((1000,), 12)


# ---- FSDP layouts ------------------------------------------------------------------------------
@pytest.mark.parametrize("n,W", [(9, 4), (10, 4), (12, 4), (1, 3), (5, 8), (100_003, 12)])
def test_fsdp1_shard_and_pad(n, W):
    flat = torch.arange(1, n + 1, dtype=torch.float32)
    S = math.ceil(n / W)
    shards = [oracle.fsdp1_get_shard(flat, r, W) for r in range(W)]
    for r, sh in enumerate(shards):
        assert sh.numel() == S
        for j in range(S):
            i = r * S + j
            assert sh[j].item() == (flat[i].item() if i < n else 0.0)
    padded = oracle.fsdp1_pad_grad(flat, W)
    assert padded.numel() == W * S and torch.equal(padded[:n], flat) and not padded[n:].any()
    assert torch.equal(oracle.gather(shards), padded)  # gather of the shards == padded flat param


@pytest.mark.parametrize("W", [2, 4, 8, 12])
def test_fsdp2_layout_against_loops(W):
    shapes = [(37, 6), (5,), (3, 2, 2), (W + 1, 3), (64, 4)]
    g = torch.Generator().manual_seed(W)
    params = [torch.randn(*s, generator=g) for s in shapes]
    n = [oracle.fsdp2_padded_shard_numel(s, W) for s in shapes]
    assert n == [math.ceil(s[0] / W) * math.prod(s[1:]) for s in shapes]
    packed = oracle.fsdp2_pack_shards(params, W)
    # index-by-index definition
    for r in range(W):
        off = 0
        for p, s in zip(params, shapes):
            rows = math.ceil(s[0] / W)
            rest = math.prod(s[1:])
            flat = p.reshape(s[0], rest)
            for i in range(rows):
                row = r * rows + i
                got = packed[r][off + i * rest : off + (i + 1) * rest]
                assert torch.equal(got, flat[row] if row < s[0] else torch.zeros(rest))
            off += rows * rest
        assert off == packed[r].numel()
    outs = oracle.fsdp2_copy_out(oracle.gather(packed), shapes, W)
    for o, p in zip(outs, params):
        assert torch.equal(o, p)
    grads = [torch.randn(*s, generator=g).bfloat16() for s in shapes]
    rs_in = oracle.fsdp2_copy_in(grads, W, torch.float32).view(W, -1)
    want = torch.stack(oracle.fsdp2_pack_shards([x.float() for x in grads], W))
    assert torch.equal(rs_in, want)  # chunk_cat == pack of the gradients, cast to fp32
    for r in range(W):
        views = oracle.fsdp2_grad_views(rs_in[r].contiguous(), shapes, W, r)
        for v, x, s in zip(views, grads, shapes):
            rows = math.ceil(s[0] / W)
            assert torch.equal(v, x.float()[r * rows : (r + 1) * rows])


def test_publish_rules():
    acc = torch.tensor([8.0, -4.0, 1.0])
    assert torch.equal(oracle.fsdp1_publish(acc.clone(), 8.0, torch.bfloat16), torch.tensor([1.0, -0.5, 0.125]).bfloat16())
    assert torch.equal(oracle.fsdp1_publish(acc.clone(), 1.0, torch.float32), acc)  # factor <= 1: no divide
    assert torch.equal(oracle.fsdp2_average(acc.clone(), 4), acc / 4)


def _nearest_f32(exact):
    """Round an exact Fraction to binary32, nearest even, by looking at the neighbours of the
    float64-rounded guess (no floating-point arithmetic decides the result)."""
    import numpy as np
    from fractions import Fraction

    guess = np.float32(float(exact))
    candidates = {guess, np.nextafter(guess, np.float32(-np.inf)), np.nextafter(guess, np.float32(np.inf))}
    best = None
    for c in candidates:
        if not np.isfinite(c):
            continue
        err = abs(Fraction(float(c)) - exact)
        even = (int(np.array(c, dtype=np.float32).view(np.uint32)) & 1) == 0
        key = (err, 0 if even else 1)
        if best is None or key < best[0]:
            best = (key, c)
    return best[1]


@pytest.mark.parametrize("divisor", [3.0, 8.0, 12.0, 64.0, 7.0])
def test_publish_division_is_correctly_rounded(divisor, c_oracle):
    """The oracle's divide (torch CPU ``/=``) against exact rational arithmetic on samples and
    against the C restatement on a large random set incl. denormals, zeros, infinities: the end
    of minibatch divide has ONE answer per element, which the HIP kernel must reproduce (a
    multiply by a rounded reciprocal differs for divisors that are not powers of two)."""
    import numpy as np
    from fractions import Fraction

    g = torch.Generator().manual_seed(int(divisor))
    x = torch.cat([
        torch.randn(200_000, generator=g) * 1e-3,
        torch.randn(1000, generator=g) * 1e-40,  # results in the denormal range
        torch.tensor([0.0, -0.0, float("inf"), -float("inf"), 1.0, 3.0, 1e-45, 3.4e38]),
        torch.arange(1, 2000, dtype=torch.float32),
    ])
    got = oracle.fsdp2_average(x.clone(), divisor)
    via_c = x.clone()
    c_oracle.oracle_divide_f32(via_c.data_ptr(), divisor, via_c.numel())
    assert torch.equal(_bits(got), _bits(via_c))
    assert torch.equal(_bits(oracle.fsdp1_publish(x.clone(), divisor, torch.float32)), _bits(via_c))
    for i in list(range(0, 200_000, 997)) + list(range(200_000, 201_000, 13)) + list(range(201_008, x.numel(), 41)):
        xi = float(x[i])
        want = _nearest_f32(Fraction(xi) / Fraction(divisor))
        assert np.float32(got[i].item()).view(np.uint32) == np.float32(want).view(np.uint32), (i, xi)
    if divisor not in (8.0, 64.0):  # the shortcut that is NOT allowed: multiply by the rounded reciprocal
        shortcut = x * torch.tensor(1.0 / divisor, dtype=torch.float32)
        finite = torch.isfinite(x)
        assert not torch.equal(_bits(shortcut[finite]), _bits(got[finite]))
    else:  # for powers of two the reciprocal is exact and the product is the same rounding
        assert torch.equal(_bits(x * (1.0 / divisor)), _bits(got))


def test_bf16_copy_of_the_accumulation_rounds_to_nearest_even(c_oracle):
    """``acc.to(bfloat16)`` (odc/fsdp/fsdp1.py:331-335, fsdp2.py:897-899) against the integer
    rounding of the C restatement, ties and the overflow to infinity included."""
    g = torch.Generator().manual_seed(0)
    x = torch.cat([torch.randn(100_000, generator=g), torch.randn(1000, generator=g) * 1e-39,
                   torch.tensor([1.00390625, 1.01171875, 3.3895314e38, 3.4e38, -3.4e38, 0.0, -0.0])])
    out = torch.empty(x.numel(), dtype=torch.int16)
    c_oracle.oracle_narrow_bf16(out.data_ptr(), x.data_ptr(), x.numel())
    assert torch.equal(out, _bits(x.to(torch.bfloat16)))
    assert torch.isinf(x.to(torch.bfloat16)[-4:-2]).all()  # 3.4e38 rounds up to infinity
