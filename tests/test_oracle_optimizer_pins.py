"""Pins for the oracle's mixed-precision optimiser pieces (oracle/cpu_ref.c: cref_squirrel_noise5, cref_noise_2d,
cref_adamw_noise, cref_adamw_mixed, cref_adamw_f32).

The reference has these only as device code (llmc/adamw.cuh, llmc/cuda_utils.cuh:238-278), which cannot be compiled
here, so each function is fixed by something that does not restate its own formula:
  * SquirrelNoise5: known answers worked through by hand from the published constants (every intermediate value is
    written out below), and what the construction guarantees whatever the constants' values: each of its eleven steps is
    a bijection of the 32-bit words (odd multiplier, addition, xor with a right shift), so the whole map is one, with
    an inverse that can be written down, and it mixes (avalanche).
  * the noise word of element i of slice s: a walk over the reference's launch grid (blockIdx.x, blockIdx.y,
    threadIdx.x as llmc/adamw.cuh:79-86 launches them and llmc/cuda_utils.cuh:272 indexes them).
  * the mixed-precision update: its fp32 state must be bit for bit that of the fp32 update on the widened inputs, its
    low-precision parameter the stochastic rounding of that state with the element's noise word; the fp32 update
    itself is held to the plain AdamW of train_gpt2.c:1007-1033 (pinned against the compiled reference in
    test_oracle_vs_reference.py) over several steps with non-zero state, decay and gradient scale.
  * the two helpers every optimiser check leans on: cref_f32_to_bf16[_array] (round to nearest even, quiet NaNs)
    against an independent cast, ties and special values included; cref_sum_squares against a float64 sum and a
    closed form.
"""
import numpy as np

import oracle_lib as ol

M32 = 0xFFFFFFFF


# ---------------------------------------------------------------------------------------------------------------------
# SquirrelNoise5
# ---------------------------------------------------------------------------------------------------------------------
# position, seed, then the word after each of the eleven steps of llmc/cuda_utils.cuh:245-255:
#   *= 0xd2a80a3f, += seed, ^= >>9, += 0xa884f197, ^= >>11, *= 0x6C736F4B, ^= >>13, += 0xB79F3ABB, ^= >>15,
#   *= 0x1b56c4f5, ^= >>17
# e.g. row 1: 0*c = 0, +0 = 0, 0^0 = 0, +0xa884f197, 0xa884f197 >> 11 = 0x0015109e and a884f197 ^ 0015109e = a891e109, ...
WORKED = [
    (0x00000000, 0x00000000, [0x00000000, 0x00000000, 0x00000000, 0xa884f197, 0xa891e109, 0x865ad4a3, 0x865ee675,
                              0x3dfe2130, 0x3dfe5acc, 0x1679153c, 0x16791e00]),
    (0x00000001, 0x00000000, [0xd2a80a3f, 0xd2a80a3f, 0xd2c15e3a, 0x7b464fd1, 0x7b492718, 0x8629dc08, 0x862ded46,
                              0x3dcd2801, 0x3dcd539b, 0xc895af57, 0xc895cb1d]),
    (0x00000000, 0x00000001, [0x00000000, 0x00000001, 0x00000001, 0xa884f198, 0xa891e106, 0x410086c2, 0x41028ec6,
                              0xf8a1c981, 0xf8a038c2, 0x23f6d9aa, 0x23f6c851]),
    (0x00000007, 0x12345678, [0xc29847b9, 0xd4cc9e31, 0xd4a6f87e, 0x7d2bea15, 0x7d244f68, 0xf3c95b78, 0xf3cec532,
                              0xab6dffed, 0xab6ca936, 0xcaaf48ae, 0xcaaf2df9]),
    (0xffffffff, 0xdeadbeef, [0x2d57f5c1, 0x0c05b4b0, 0x0c03b66a, 0xb488a801, 0xb49e3914, 0x991664dc, 0x9912ac6f,
                              0x50b1e72a, 0x50b14649, 0x42fe27dd, 0x42fe06a2]),
]


def test_squirrel_noise5_known_answers():
    L = ol.cref()
    for pos, seed, trail in WORKED:
        assert L.cref_squirrel_noise5(pos, seed) == trail[-1], (hex(pos), hex(seed))
    # the trails are self-consistent where a step is linear in the seed: seed enters by one addition after the first
    # multiplication, so equal (pos*c + seed) gives equal output
    c = 0xd2a80a3f
    for pos in (3, 1000, 0x80000001):
        a = L.cref_squirrel_noise5(pos, 5)
        b = L.cref_squirrel_noise5(0, (pos * c + 5) & M32)
        assert a == b


def _unxorshift(y, s):
    x = y
    for _ in range(32 // s + 1):
        x = y ^ (x >> s)
    return x


def _sq5_inverse(y, seed):
    """Undo the eleven steps in reverse order with modular inverses and xorshift inversion."""
    inv = lambda c: pow(c, -1, 1 << 32)
    x = _unxorshift(y, 17)
    x = (x * inv(0x1b56c4f5)) & M32
    x = _unxorshift(x, 15)
    x = (x - 0xB79F3ABB) & M32
    x = _unxorshift(x, 13)
    x = (x * inv(0x6C736F4B)) & M32
    x = _unxorshift(x, 11)
    x = (x - 0xa884f197) & M32
    x = _unxorshift(x, 9)
    x = (x - seed) & M32
    return (x * inv(0xd2a80a3f)) & M32


def test_squirrel_noise5_is_a_bijection_that_mixes():
    L = ol.cref()
    rng = np.random.default_rng(5)
    # invertible: positions come back from their noise words
    for pos, seed in rng.integers(0, 1 << 32, size=(300, 2), dtype=np.uint64):
        assert _sq5_inverse(L.cref_squirrel_noise5(int(pos), int(seed)), int(seed)) == int(pos)
    # injective on a slice of 2^16 consecutive positions (a random function would collide about 0.5 times here;
    # over 2^18 positions of four slices about 8 times; a bijection never does)
    for seed, base in ((0, 0), (12345, 0xfffe0000), (0xdeadbeef, 1 << 20), (7, 0x7fff8000)):
        words = {L.cref_squirrel_noise5((base + i) & M32, seed) for i in range(1 << 16)}
        assert len(words) == 1 << 16
    # avalanche: flipping one input bit flips about half of the output bits (binomial(32, 1/2) per trial; the mean
    # over 32 bits x 200 positions stays within 16 +- 1 and every single input bit moves at least a quarter of them)
    flips = np.zeros(32)
    n = 200
    for pos in rng.integers(0, 1 << 32, size=n, dtype=np.uint64):
        w = L.cref_squirrel_noise5(int(pos), 99)
        for b in range(32):
            flips[b] += bin(w ^ L.cref_squirrel_noise5(int(pos) ^ (1 << b), 99)).count("1")
    flips /= n
    assert abs(flips.mean() - 16.0) < 1.0, flips.mean()
    assert flips.min() > 8.0, flips
    # and the low 16 bits, the ones the rounding threshold is taken from, are uniform: chi-square over 256 bins
    lows = np.array([L.cref_squirrel_noise5(i, 2024) & 0xffff for i in range(1 << 16)])
    hist = np.bincount(lows >> 8, minlength=256)
    chi2 = ((hist - 256.0) ** 2 / 256.0).sum()
    assert chi2 < 400.0, chi2         # 255 degrees of freedom: mean 255, sd 22.6


def test_noise_2d_is_the_prime_walk():
    L = ol.cref()
    # Get2dNoiseUint(x, y, seed) = SquirrelNoise5(x + 198491317*y) (llmc/cuda_utils.cuh:257-264): y advances the
    # position by the prime, so (x + P, y) and (x, y + 1) name the same word, and y = 0 is the 1-d noise
    P = 198491317
    for x, y, seed in ((0, 0, 1), (5, 7, 11), (511, 70000, 3), (100, 2 ** 31 - 1, 4)):
        assert L.cref_noise_2d(x, y, seed) == L.cref_squirrel_noise5((x + P * y) & M32, seed)
        assert L.cref_noise_2d(x, 0, seed) == L.cref_squirrel_noise5(x, seed)
    assert L.cref_noise_2d(3 + P, 9, 8) == L.cref_noise_2d(3, 10, 8)


# ---------------------------------------------------------------------------------------------------------------------
# the noise word of an element under the reference's launch geometry
# ---------------------------------------------------------------------------------------------------------------------
def test_adamw_noise_walks_the_reference_grid():
    L = ol.cref()
    n, slices, seed, block = 1500, 3, 0xabcdef, 512
    grid_x = -(-n // block)                                  # CEIL_DIV(num_parameters, block_size), adamw.cuh:80
    table = {}
    for bx in range(grid_x):                                 # dim3(num_blocks, num_slices) x block_size, adamw.cuh:83
        for by in range(slices):
            for tx in range(block):
                idx = bx * block + tx                        # adamw.cuh:22
                if idx >= n:
                    continue                                 # adamw.cuh:23
                # stochastic_rounding: Get2dNoiseUint(threadIdx.x, blockIdx.x * blockDim.x + blockIdx.y, seed)
                table[(idx, by)] = L.cref_noise_2d(tx, bx * block + by, seed)
    assert len(table) == n * slices
    for (idx, by), want in table.items():
        assert L.cref_adamw_noise(idx, by, seed) == want, (idx, by)
    # the words of one slice are not all distinct from the next slice's (block b of slice s+1 reuses y = 512b + s + 1),
    # but inside a slice no two elements share a position
    for by in range(slices):
        pos = {((idx % 512) + 198491317 * ((idx // 512) * 512 + by)) & M32 for idx in range(n)}
        assert len(pos) == n


# ---------------------------------------------------------------------------------------------------------------------
# AdamW
# ---------------------------------------------------------------------------------------------------------------------
def _rnd(n, seed, scale=1.0):
    return (np.random.default_rng(seed).standard_normal(n) * scale).astype(np.float32)


def test_adamw_f32_tracks_plain_adamw_over_steps():
    # cref_adamw is train_gpt2.c's loop (pinned against the compiled reference's gpt2_update on a whole model); the
    # lerp form (llmc/adamw.cuh:14-16, 27-31) must give the same trajectory up to fp32 rounding, with decay, with
    # state carried over steps, and grad_scale folded into the gradient
    L = ol.cref()
    n, lr, b1, b2, eps, wd = 1003, 3e-3, 0.9, 0.95, 1e-8, 0.1
    p = _rnd(n, 0); m = np.zeros(n, np.float32); v = np.zeros(n, np.float32)
    p2 = p.copy(); m2 = m.copy(); v2 = v.copy()
    p3 = p.copy(); m3 = m.copy(); v3 = v.copy(); ms3 = p.copy()
    for t in range(1, 7):
        g = _rnd(n, 10 + t, 0.3)
        L.cref_adamw(p, m, v, (0.5 * g).astype(np.float32), n, lr, b1, b2, eps, wd, t)
        L.cref_adamw_f32(p2, None, g, m2, v2, n, lr, b1, b2, t, eps, wd, 0.5)
        L.cref_adamw_f32(p3, ms3.ctypes.data, g, m3, v3, n, lr, b1, b2, t, eps, wd, 0.5)
        np.testing.assert_allclose(m2, m, rtol=2e-6, atol=1e-9)
        np.testing.assert_allclose(v2, v, rtol=2e-6, atol=1e-12)
        np.testing.assert_allclose(p2, p, rtol=0, atol=2e-6 * t)
        # with fp32 parameters the master copy is the parameter
        assert np.array_equal(p3, p2) and np.array_equal(ms3, p2) and np.array_equal(m3, m2) and np.array_equal(v3, v2)
    # a transposed lerp (weights of m and g exchanged) or a missing bias correction is far outside these bounds:
    wrong_m = (1 - b1) * m + b1 * (0.5 * g)
    assert np.abs(wrong_m - m).max() > 1e-2


def test_adamw_mixed_is_the_f32_update_plus_stochastic_rounding():
    L = ol.cref()
    n, lr, b1, b2, eps, wd, gs, seed = 1500, 1e-2, 0.9, 0.95, 1e-8, 0.1, 0.7, 4242
    for use_master in (True, False):
        for slice_ in (0, 2):
            g32 = _rnd(n, 1, 0.5); gb = np.zeros(n, np.uint16); L.cref_f32_to_bf16_array(gb, g32, n)
            gw = np.zeros(n, np.float32); L.cref_bf16_to_f32_array(gw, gb, n)           # the gradients as the update sees them
            p32 = _rnd(n, 2); pb = np.zeros(n, np.uint16); L.cref_f32_to_bf16_array(pb, p32, n)
            pw = np.zeros(n, np.float32); L.cref_bf16_to_f32_array(pw, pb, n)
            master = (pw + _rnd(n, 3, 1e-3)).astype(np.float32)                          # differs from the bf16 copy
            m = _rnd(n, 4, 0.1); v = np.abs(_rnd(n, 5, 0.01))
            # fp32 leg on the widened inputs
            fp = (master if use_master else pw).copy(); fm = m.copy(); fv = v.copy()
            L.cref_adamw_f32(fp, None, gw, fm, fv, n, lr, b1, b2, 3, eps, wd, gs)
            # mixed leg
            mp = pb.copy(); mm = m.copy(); mv = v.copy(); mms = master.copy()
            L.cref_adamw_mixed(mp, mms.ctypes.data if use_master else None, gb, mm, mv, n, lr, b1, b2, 3, eps, wd, gs,
                               seed, slice_)
            assert np.array_equal(mm.view(np.uint32), fm.view(np.uint32))
            assert np.array_equal(mv.view(np.uint32), fv.view(np.uint32))
            if use_master:
                assert np.array_equal(mms.view(np.uint32), fp.view(np.uint32))
            else:
                assert np.array_equal(mms, master)                                       # untouched
            want = np.array([L.cref_stochastic_round_bf16(float(fp[i]), L.cref_adamw_noise(i, slice_, seed))
                             for i in range(n)], np.uint16)
            assert np.array_equal(mp, want)
            # and the rounding is a rounding: each parameter is one of the two bf16 neighbours of the fp32 value
            lo = (fp.view(np.uint32) >> 16).astype(np.uint32)
            got = mp.astype(np.uint32)
            assert np.all((got == lo) | (got == lo + 1))
            assert 0.2 < np.mean(got == lo + 1) < 0.8                                    # both neighbours occur


# ---------------------------------------------------------------------------------------------------------------------
# cref_sum_squares and cref_f32_to_bf16[_array]: the two helpers the optimiser tests lean on
# ---------------------------------------------------------------------------------------------------------------------
def test_sum_squares_is_the_double_precision_sum():
    """dev/cuda/global_norm.cu:21-28 accumulates in double. Checked against numpy's float64 sum, on inputs where a
    float accumulator is visibly off: 300000 values of 1 + 2^-12 k/n summed in fp32 lose the 6th digit."""
    L = ol.cref()
    n = 300000
    x = (1.0 + np.arange(n, dtype=np.float64) / n * 2.0 ** -12).astype(np.float32)
    want = float(np.sum(x.astype(np.float64) ** 2))
    got = L.cref_sum_squares(x, n)
    assert abs(got - want) <= 1e-12 * want
    naive = float(np.cumsum((x * x).astype(np.float32), dtype=np.float32)[-1])
    assert abs(naive - want) > 1e-6 * want                              # the case separates float from double
    # signs, magnitudes 1e-20 ... 1e+18 and a closed form: sum of k^2 for k = 1..n is n(n+1)(2n+1)/6
    r = np.random.default_rng(5)
    y = (r.standard_normal(100003) * 10.0 ** r.uniform(-20, 18, 100003)).astype(np.float32)
    want = float(np.sum(y.astype(np.float64) ** 2))
    assert abs(L.cref_sum_squares(y, y.size) - want) <= 1e-12 * want
    k = np.arange(1, 2001, dtype=np.float32)
    assert L.cref_sum_squares(k, k.size) == 2000 * 2001 * 4001 / 6
    assert L.cref_sum_squares(k, 0) == 0.0


def test_f32_to_bf16_rounds_to_nearest_even_like_the_library_cast():
    """__float2bfloat16_rn (what the reference's (floatX) casts compile to, llmc/cuda_common.h:82-92) is IEEE
    round-to-nearest-even with quiet NaNs. Checked against torch's cast (an independent implementation) on random bit
    patterns and on the cases a rounding mistake shows in: every exact tie of several exponents with both parities of
    the kept bit, the values one unit either side of a tie, +-0, +-inf, denormals, the carry into the exponent and
    into infinity, NaNs."""
    import torch
    L = ol.cref()
    r = np.random.default_rng(11)
    bits = [r.integers(0, 2 ** 32, 1 << 20, dtype=np.uint64).astype(np.uint32)]
    for e in (0, 1, 37, 126, 127, 128, 200, 254):                       # exponent fields incl. denormal and the largest
        for sign in (0, 1):
            hi = (np.arange(128, dtype=np.uint32) | np.uint32(e << 7) | np.uint32(sign << 15)) << 16  # all 7-bit mantissas
            for low in (0x0000, 0x0001, 0x7fff, 0x8000, 0x8001, 0xffff):
                bits.append(hi | np.uint32(low))
    bits.append(np.array([0x00000000, 0x80000000, 0x7f800000, 0xff800000, 0x00000001, 0x80000001, 0x007fffff,
                          0x7f7fffff, 0xff7fffff, 0x7f7f8000, 0x7f7f7fff, 0x3f7fffff, 0x3f7f8000], np.uint32))
    bits = np.concatenate(bits)
    x = bits.view(np.float32)
    got = np.zeros(x.size, np.uint16)
    L.cref_f32_to_bf16_array(got, x, x.size)
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    nan = (bits & 0x7fffffff) > 0x7f800000          # a NaN's payload is the implementation's choice: both must be NaN
    assert nan.sum() > 1000 and np.array_equal(got[~nan], want[~nan])
    assert np.all((got[nan] & 0x7f80) == 0x7f80) and np.all((got[nan] & 0x7f) != 0)
    assert np.all((want[nan] & 0x7f80) == 0x7f80) and np.all((want[nan] & 0x7f) != 0)
    # ties by hand: 1 + 2^-8 lies midway between 1 (kept bit 0) and 1 + 2^-7 -> down; 1 + 3*2^-8 -> up to 1 + 2^-6
    assert L.cref_f32_to_bf16(np.float32(1 + 2.0 ** -8)) == 0x3f80
    assert L.cref_f32_to_bf16(np.float32(1 + 3 * 2.0 ** -8)) == 0x3f82
    assert L.cref_f32_to_bf16(np.float32(3.3895313892515355e38)) == 0x7f7f                 # largest bf16, exact
    assert L.cref_f32_to_bf16(np.float32(3.4028234663852886e38)) == 0x7f80                 # FLT_MAX rounds to inf
    # NaNs stay NaNs (quiet), whatever their payload, and keep their sign
    nan_bits = np.array([0x7fc00000, 0x7f800001, 0x7f80ffff, 0xffc00000, 0xff800001, 0x7fffffff, 0x7fa00000], np.uint32)
    out = np.zeros(nan_bits.size, np.uint16)
    L.cref_f32_to_bf16_array(out, nan_bits.view(np.float32), nan_bits.size)
    assert np.all((out & 0x7f80) == 0x7f80) and np.all((out & 0x007f) != 0)
    assert np.array_equal(out >> 15, (nan_bits >> 31).astype(np.uint16))
    # scalar and array forms agree, and widening is the inverse on representable values
    # (not on denormals: the scalar crosses ctypes as a double narrowed to float, which flushes them to zero once a
    # library built with fast-math flags, such as the compiled reference, has been loaded into the process)
    for i in range(0, x.size, 9973):
        if (bits[i] & 0x7f800000) != 0 and not nan[i]:
            assert L.cref_f32_to_bf16(x[i]) == got[i]
    h = r.integers(0, 2 ** 16, 4096, dtype=np.uint32).astype(np.uint16)
    h = h[(h & 0x7f80) != 0x7f80]
    wide = np.zeros(h.size, np.float32); L.cref_bf16_to_f32_array(wide, h, h.size)
    back = np.zeros(h.size, np.uint16); L.cref_f32_to_bf16_array(back, wide, h.size)
    assert np.array_equal(back, h) and np.array_equal(wide.view(np.uint32), h.astype(np.uint32) << 16)
