"""Pins the oracle's append path (encode, cluster counts, query prep) against
closed forms and library routines.  CPU only."""
import json
import os

import numpy as np
import pytest
import scipy.linalg
import torch

import refforms

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def test_bf16_round_matches_torch(oracle):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(100000, generator=g) * torch.exp(torch.randn(100000, generator=g) * 8)
    x = torch.cat([x, torch.tensor([0.0, -0.0, 1.0, 65504.0, 3.3895e38, 1e-40, float("inf")])])
    ref = x.to(torch.bfloat16).float().numpy()
    assert np.array_equal(oracle.bf16_round(x.numpy()).view(np.uint32), ref.view(np.uint32))
    for v in x[:2000].tolist():
        assert np.float32(oracle.lib().pkv_o_bf16_round(v)).view(np.uint32) == np.float32(
            torch.tensor(v).to(torch.bfloat16).float().item()).view(np.uint32)


def test_mag_constants_match_torch_and_reference_data(oracle):
    th, ce = oracle.mag_constants()
    assert np.array_equal(th, torch.tensor(refforms.MAG_THRESHOLDS, dtype=torch.bfloat16).float().numpy())
    assert np.array_equal(ce, torch.tensor(refforms.MAG_CENTERS, dtype=torch.bfloat16).float().numpy())
    # known bf16 values
    assert th.tolist() == [0.08447265625, 0.169921875, 0.2578125, 0.349609375, 0.44921875, 0.55859375, 0.69140625]
    assert ce.tolist() == [0.0419921875, 0.126953125, 0.212890625, 0.302734375, 0.396484375, 0.5, 0.6171875, 0.76171875]
    # the literals agree with the reference's Lloyd-Max data file to Monte-Carlo noise
    data = json.load(open(os.path.join(GOLD, "magnitude_levels_m8_4bit.json")))
    np.testing.assert_allclose(data["thresholds"], refforms.MAG_THRESHOLDS, atol=5e-4)
    np.testing.assert_allclose(data["centers"], refforms.MAG_CENTERS, atol=5e-4)


def test_sign_codebook_is_bit_enumeration():
    cb = json.load(open(os.path.join(GOLD, "codebook_d128_m8_Kr1_Kw256_rabitq_sign.json")))
    assert cb["config"]["d"] == 128 and cb["config"]["m"] == 8 and cb["config"]["K_omega"] == 256
    s = np.array(cb["angular_signs"])
    for c in range(256):
        for j in range(8):
            assert (s[c, j] > 0) == bool((c >> j) & 1)


def test_philox_known_answers_and_srht_signs(oracle):
    """The SRHT sign vector is a Philox4x32-10 draw (the generator behind torch's device RNG).  The block function is
    pinned by the three known-answer vectors of the Random123 distribution (zeros, ones, digits of pi); the sign
    vector by its definition from the block function, by the product's independent host restatement, and by
    balance (a gross indexing error would not give 128 fair coin flips from 128 counters)."""
    kat = [((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
           ((0xffffffff,) * 4, (0xffffffff,) * 2, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
           ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
            (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1))]
    for ctr, key, want in kat:
        assert tuple(oracle.philox4x32_10(ctr, key)) == want
    from pariskv_amd import ops

    for seed in (42, 0, 123456789012):
        s = oracle.srht_signs(seed)
        assert s.dtype == np.float32 and s.shape == (128,) and set(np.unique(s)) == {-1.0, 1.0}
        assert [oracle.philox4x32_10((0, 0, i, 0), (seed & 0xffffffff, seed >> 32))[0] % 2 for i in range(128)] == \
            [int(x > 0) for x in s]
        assert np.array_equal(ops.srht_signs("cpu", seed).numpy(), s)
        assert 40 <= int((s > 0).sum()) <= 88
    assert oracle.srht_signs(42)[:12].tolist() == [1, 1, -1, -1, 1, 1, -1, -1, -1, 1, 1, 1]


def test_fwht_matches_hadamard_matrix(oracle):
    H = scipy.linalg.hadamard(128).astype(np.float64)
    g = np.random.default_rng(0)
    xi = g.integers(-50, 50, size=(64, 128)).astype(np.float32)  # exact in fp32
    assert np.array_equal(oracle.fwht128(xi), (xi.astype(np.float64) @ H).astype(np.float32))
    x = g.standard_normal((64, 128)).astype(np.float32)
    y = oracle.fwht128(x)
    err = np.abs(y - x.astype(np.float64) @ H)
    assert (err <= 2e-6 * np.abs(x).sum(axis=1, keepdims=True)).all()
    np.testing.assert_allclose(oracle.fwht128(y) / 128.0, x, atol=1e-5)  # involution
    e = np.zeros((1, 128), np.float32)
    e[0, 5] = 1.0
    assert np.array_equal(oracle.fwht128(e)[0], H[5].astype(np.float32))  # row of H, natural order


@pytest.mark.parametrize("dtype_name", ["f32", "bf16"])
def test_encode_matches_library_restatement(oracle, signs, dtype_name):
    bf = dtype_name == "bf16"
    keys = oracle.synth_keys(6000, seed=3, bf16=bf)
    codes, nib, w = oracle.encode(keys, signs, oracle.BF16 if bf else oracle.F32)
    tk = torch.from_numpy(keys)
    if bf:
        tk = tk.to(torch.bfloat16)
    rc, rp, rw = refforms.batch_encode(tk, torch.from_numpy(signs))
    rc, rp, rw = rc.numpy(), rp.numpy(), rw.float().numpy()
    # codes and nibbles hinge on fp32 round-off only where a rotated coordinate
    # or a direction sits on a boundary: near-total agreement is the pin
    assert (codes == rc).mean() > 0.9995
    assert (nib == rp).mean() > 0.995
    agree = (nib == rp).all(axis=2)
    rel = np.abs(w - rw) / np.maximum(np.abs(rw), 1e-6)
    assert np.median(rel) == 0.0 or np.median(rel) < 1e-2
    assert rel[agree].max() <= 2 ** -7  # at most one bf16 ulp where the codes agree
    # ... and bit-identical almost everywhere: what is left is the summation order inside torch's reductions
    assert (w[agree] == rw[agree]).mean() >= 0.99
    # invariants
    assert w.min() > 0 and np.array_equal(oracle.bf16_round(w), w)
    assert ((nib & 0x07) <= 7).all()


def test_encode_exact_closed_form_cases(oracle):
    """Inputs for which every fp step is exact, so the codes have a closed form."""
    ones = np.ones(128, np.float32)
    # key = c * e_0 with all-ones signs: rotated vector is constant 1/sqrt(128) > 0
    k = np.zeros((1, 128), np.float32)
    k[0, 0] = 4.0
    codes, nib, w = oracle.encode(k, ones, oracle.F32)
    assert (codes == 255).all()
    # direction of each block is 1/sqrt(8)=0.3536 in every dim -> bucket 4 (0.3496 < u <= 0.4492), sign bit set
    assert (nib == ((8 | 4) << 4 | (8 | 4))).all()
    th, ce = oracle.mag_constants()
    r = np.sqrt(8.0 / 128.0)
    alpha = 8 * ce[4] * (1 / np.sqrt(8.0))
    np.testing.assert_allclose(w, np.full_like(w, oracle.bf16_round(np.float32([r / alpha * 4.0]))[0]), rtol=2 ** -7)
    # flipping the SRHT sign of dim 0 negates everything: all sign bits clear
    s = ones.copy()
    s[0] = -1
    codes2, nib2, _ = oracle.encode(k, s, oracle.F32)
    assert (codes2 == 0).all() and (nib2 == (4 << 4 | 4)).all()
    # zero key: no NaNs, codes 255 (0 >= 0), magnitude bucket 0, weight 0
    codes3, nib3, w3 = oracle.encode(np.zeros((1, 128), np.float32), ones, oracle.BF16)
    assert (codes3 == 255).all() and (nib3 == 0x88).all() and (w3 == 0).all()


def _bf16(x):
    """Round-to-nearest-even bf16 of float32 values, by integer arithmetic on the bit patterns."""
    u = np.asarray(x, np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


# keys k[i] = ((i * a) mod (2b + 3) - (b + 1)) / 4 and the bf16 bit patterns of their 16 block weights
_ALPHA_ROUNDING_KEYS = {
    (1, 1): [0x3f8f, 0x3f19, 0x3f53, 0x3f8f, 0x3f75, 0x3f39, 0x3f8a, 0x3f32, 0x3f44, 0x3f89, 0x3fa8, 0x3fa6, 0x3f77, 0x3f71,
             0x3fa8, 0x3fba],
    (4, 4): [0x3fc9, 0x4058, 0x3fc0, 0x4014, 0x4007, 0x402f, 0x3f9a, 0x4053, 0x3ff3, 0x3fb7, 0x3fea, 0x403f, 0x401f, 0x3fc8,
             0x402a, 0x4024],
    (1, 7): [0x409d, 0x4076, 0x406d, 0x403e, 0x401d, 0x4056, 0x4040, 0x4061, 0x4081, 0x4081, 0x4065, 0x40a7, 0x403b, 0x4021,
             0x404a, 0x3ff6],
}


@pytest.mark.parametrize("ab", sorted(_ALPHA_ROUNDING_KEYS))
def test_block_weight_rounds_the_alpha_products_before_the_sum(oracle, signs, ab):
    """polar_cache.py:972-976 in the bf16 chain: ``a_vals * abs_u`` is a bf16 tensor, so every product is rounded to
    bf16 BEFORE the fp32 sum that gives alpha.  These constructed keys are ones where that rounding point shows in
    the stored weight: summing the unrounded products changes the bf16 bits of at least three blocks.  The expected
    bits are written out above; they are what torch produces for the reference's own expression, and what the
    restatement below (numpy, bf16 rounding by integer arithmetic, independent of the oracle's code) gives with the
    rounding in place."""
    a, b = ab
    key = np.array([(((i * a) % (2 * b + 3)) - (b + 1)) * 0.25 for i in range(128)], np.float32)  # exact in bf16
    expected = np.array(_ALPHA_ROUNDING_KEYS[ab], np.uint16)
    _, _, w = oracle.encode(key[None], signs, oracle.BF16)
    got = (w[0].view(np.uint32) >> 16).astype(np.uint16)
    assert np.array_equal(got, expected), [hex(x) for x in got]
    # the reference's torch expression on the same key
    _, _, rw = refforms.batch_encode(torch.from_numpy(key).to(torch.bfloat16)[None], torch.from_numpy(signs))
    assert np.array_equal(rw.view(torch.int16).numpy()[0].astype(np.uint16), expected)
    # independent restatement from the rotated vector on, with and without the rounding of the products
    th, ce = oracle.mag_constants()
    n = _bf16(np.sqrt(np.float32((key.astype(np.float64) ** 2).sum())))
    x = _bf16(key / n) * signs
    y = _bf16((x.astype(np.float64) @ scipy.linalg.hadamard(128)).astype(np.float32) * np.float32(1 / np.sqrt(128.0)))
    rounded, unrounded = [], []
    for blk in y.reshape(16, 8):
        r = _bf16(np.sqrt(np.float32((blk.astype(np.float64) ** 2).sum())))
        au = np.abs(_bf16(blk / r))
        t = (th[None, :] < au[:, None]).sum(axis=1)
        prod = (ce[t] * au).astype(np.float32)
        for out, terms in ((rounded, _bf16(prod)), (unrounded, prod)):
            alpha = np.float32(0)
            for p in terms:
                alpha = np.float32(alpha + p)
            out.append(_bf16(np.float32(np.float32(r / max(alpha, np.float32(1e-6))) * n)))
    rounded = (np.array(rounded, np.float32).view(np.uint32) >> 16).astype(np.uint16)
    unrounded = (np.array(unrounded, np.float32).view(np.uint32) >> 16).astype(np.uint16)
    assert np.array_equal(rounded, expected)
    assert (unrounded != expected).sum() >= 3


def test_bf16_quotients_stay_clear_of_bf16_rounding_boundaries(oracle):
    """What the GPU encoder's reciprocal path rests on: for bf16 operands the quotient x / d is never within a
    relative 2^-18 of a bf16 rounding boundary (the midpoint of two neighbouring bf16 numbers) unless it is exactly
    a bf16 number, so any fp32 value within 2^-21 of the quotient rounds to the same bf16 as the correctly rounded
    fp32 quotient does.  Exhaustive over the 128 x 128 significand pairs (the exponents only scale the picture)."""
    from fractions import Fraction
    closest = Fraction(1)
    for mx in range(128, 256):
        for md in range(128, 256):
            q = Fraction(mx, md)
            half_ulp_den = 256 if q >= 1 else 512           # boundaries are odd multiples of 1/256 in [1, 2), of 1/512 in (1/2, 1)
            k = (q * half_ulp_den - 1) / 2                   # q = (2k + 1) / den  <=>  k integer
            lo, hi = Fraction(2 * int(k) + 1, half_ulp_den), Fraction(2 * int(k) + 3, half_ulp_den)
            dist = min(abs(q - lo), abs(q - hi)) / q
            assert dist != 0, (mx, md)
            closest = min(closest, dist)
    assert closest > Fraction(1, 1 << 18)
    # the same statement as arithmetic: perturb every quotient by +-2^-21 (more than a 1-ulp reciprocal times a
    # rounded product can be off) at several exponents and round as the kernel does
    mx, md = np.meshgrid(np.arange(128, 256, dtype=np.float64), np.arange(128, 256, dtype=np.float64), indexing="ij")
    for ex, ed in ((0, 0), (-20, 3), (7, -9), (-3, 30)):
        x, d = (mx * 2.0 ** (ex - 7)).astype(np.float32), (md * 2.0 ** (ed - 7)).astype(np.float32)
        want = oracle.bf16_round(x / d)                      # fp32 division, correctly rounded, then bf16
        for eps in (-2.0 ** -21, 2.0 ** -21):
            approx = ((x.astype(np.float64) / d.astype(np.float64)) * (1.0 + eps)).astype(np.float32)
            assert np.array_equal(oracle.bf16_round(approx).view(np.uint32), want.view(np.uint32))


def test_encode_brute_force_nearest_sign_centroid(oracle, signs):
    """Sign bit-pack == argmax over the 256 sign centroids of <V_c, y_b>."""
    keys = oracle.synth_keys(300, seed=11)
    codes, _, _ = oracle.encode(keys, signs, oracle.F32)
    V = np.array([[1.0 if (c >> j) & 1 else -1.0 for j in range(8)] for c in range(256)])
    y = (keys / np.linalg.norm(keys, axis=1, keepdims=True) * signs) @ scipy.linalg.hadamard(128) / np.sqrt(128)
    best = (y.reshape(-1, 16, 8) @ V.T).argmax(axis=-1)
    assert (best == codes).mean() > 0.9999


def test_nibble_pack_roundtrip_exhaustive():
    allb = torch.arange(256, dtype=torch.uint8).view(-1, 1).repeat(1, 4)
    s, t = refforms.unpack_4bit(allb)
    assert torch.equal(refforms.pack_4bit(s > 0, t.to(torch.uint8)), allb)


def test_count_cluster_keys_is_bincount(oracle):
    g = np.random.default_rng(5)
    codes = g.integers(0, 256, size=(5000, 16), dtype=np.uint8)
    counts = oracle.count_cluster_keys(codes)
    for b in range(16):
        assert np.array_equal(counts[b], np.bincount(codes[:, b], minlength=256))
    more = oracle.count_cluster_keys(codes[:100], counts.copy())  # accumulates (polar_cache.py:774-775)
    assert more.sum() == counts.sum() + 1600


@pytest.mark.parametrize("dtype_name", ["f32", "bf16"])
def test_query_prep_matches_library_restatement(oracle, signs, dtype_name):
    bf = dtype_name == "bf16"
    keys = oracle.synth_keys(512, seed=7, bf16=bf)
    bad = 0
    for s in range(20):
        q = oracle.synth_queries(keys, 4, seed=s, bf16=bf)
        qhat, qn = oracle.query_prep(q, signs, oracle.BF16 if bf else oracle.F32)
        tq = torch.from_numpy(q).to(torch.bfloat16 if bf else torch.float32)
        rh, rn = refforms.encode_query(tq, torch.from_numpy(signs))
        tol = 2 ** -7 if bf else 1e-5
        assert abs(qn - float(rn)) <= tol * abs(float(rn))
        np.testing.assert_allclose(qhat, rh.float().numpy(), rtol=0, atol=tol)
        bad += int((qhat != rh.float().numpy()).sum())
        assert abs(np.linalg.norm(qhat.astype(np.float64)) - 1.0) < (2e-2 if bf else 1e-5)  # rotation keeps the unit norm
    if bf:  # bf16 rounding hides the summation order except at rounding boundaries
        assert bad <= 20 * 128 * 0.02


def test_one_instruction_butterfly_stages_carry_only_a_sign(oracle):
    """The encoder's lane-crossing Walsh-Hadamard stages as the HIP kernel runs them, simulated in float32: block s of
    a key sits in lane s0*1 ^ s1*2 ^ s2*7 ^ s3*15 (every partner then is one lane-permute move away), a stage is
    held' = held[partner] * c + held with c = -1 where the block's stage bit is set, and what is left is the sign
    (-1)^(set bits of s), taken out by the sign of the final scale.  Bit for bit the natural butterfly
    (t + o where the bit is clear, o - t where it is set) followed by the plain scale."""
    lane_of = lambda s: ((s & 1) * 1) ^ (((s >> 1) & 1) * 2) ^ (((s >> 2) & 1) * 7) ^ (((s >> 3) & 1) * 15)
    lanes = [lane_of(s) for s in range(16)]
    assert sorted(lanes) == list(range(16))                                   # a placement: every lane holds one block
    block_of = lambda l: l ^ (3 if l & 4 else 0) ^ (4 if l & 8 else 0)        # the kernel's inverse map
    assert all(block_of(lane_of(s)) == s for s in range(16))
    partner_xor = {1: 1, 2: 2, 4: 7, 8: 15}                                   # quad_perm, quad_perm, row_half_mirror, row_mirror
    for bit, x in partner_xor.items():
        assert all(lane_of(s ^ bit) == lane_of(s) ^ x for s in range(16))
    rng = np.random.default_rng(7)
    scale = np.float32(0.08838834764831845)
    for trial in range(200):
        v = (rng.standard_normal(16) * np.exp2(rng.integers(-20, 20))).astype(np.float32)
        if trial % 5 == 0:
            v[rng.integers(0, 16, size=4)] = v[0]                            # equal pairs: exact zeros on the way
        # natural form, block s in slot s
        t = v.copy()
        for bit in (1, 2, 4, 8):
            o = t[np.arange(16) ^ bit]
            t = np.where(np.arange(16) & bit, o - t, t + o).astype(np.float32)
        want = (t * scale).astype(np.float32)
        # the kernel's form, in lanes
        held = np.empty(16, np.float32)
        for s in range(16):
            held[lane_of(s)] = v[s]
        blocks = np.array([block_of(l) for l in range(16)])
        for bit, x in partner_xor.items():
            c = np.where(blocks & bit, np.float32(-1), np.float32(1)).astype(np.float32)
            prod = (held[np.arange(16) ^ x] * c).astype(np.float32)          # exact: c is +-1, so the fused form rounds once
            held = (prod + held).astype(np.float32)
        parity = np.array([bin(b).count("1") & 1 for b in blocks])
        got_lanes = (held * np.where(parity, -scale, scale).astype(np.float32)).astype(np.float32)
        got = np.array([got_lanes[lane_of(s)] for s in range(16)], np.float32)
        nz = want != 0                                                        # zeros take the kernel's exact path
        assert np.array_equal(got[nz].view(np.uint32), want[nz].view(np.uint32)), trial
        assert np.all(got[~nz] == 0)


def _rn32(fr):
    """A rational rounded to the nearest float32 (ties to even), as a Fraction; normal range only."""
    from fractions import Fraction
    if fr == 0:
        return Fraction(0)
    sign, a = (-1 if fr < 0 else 1), abs(fr)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1                                            # 2^e <= a < 2^(e+1)
    q = a / Fraction(2) ** (e - 23)                       # in [2^23, 2^24)
    n = q.numerator // q.denominator
    rem = q - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and n & 1):
        n += 1
    return sign * n * Fraction(2) ** (e - 23)


def test_shared_reciprocal_division_and_unscaled_root_are_correctly_rounded():
    """What the GPU encoder's fp32 chain rests on, in exact rational arithmetic: from ANY reciprocal estimate within
    one ulp, one Newton step and two residual corrections (each a fused multiply-add, rounded once) give the
    correctly rounded quotient, and the hardware root (within one ulp) moved by the signs of two residuals gives the
    correctly rounded root.  The refined reciprocal depends on the denominator alone, so eight quotients share it."""
    from fractions import Fraction
    rng = np.random.default_rng(11)
    F = lambda v: Fraction(float(v))
    fma = lambda a, b, c: _rn32(a * b + c)
    ulp = lambda v: Fraction(2) ** ((v.numerator.bit_length() - v.denominator.bit_length() - (Fraction(2) ** (v.numerator.bit_length() - v.denominator.bit_length()) > v)) - 23)
    dens = np.concatenate([rng.uniform(1.0, 2.0, 300), [1.0, 1.5, 2.0 - 2.0 ** -23, 1.0 + 2.0 ** -23]]).astype(np.float32)
    for d32 in dens:
        d = F(d32) * Fraction(2) ** int(rng.integers(-20, 40))
        for off in (-1, 0, 1):                            # the reciprocal instruction: anything within one ulp
            y0 = _rn32(1 / d)
            y0 = y0 + off * ulp(y0)
            y = fma(fma(-d, y0, Fraction(1)), y0, y0)
            for a32 in rng.uniform(-2.0, 2.0, 6).astype(np.float32):
                a = F(a32) * Fraction(2) ** int(rng.integers(-30, 30))
                q = _rn32(a * y)
                q = fma(fma(-d, q, a), y, q)
                q = fma(fma(-d, q, a), y, q)
                assert q == _rn32(a / d), (float(a), float(d), off)
    for a32 in np.concatenate([rng.uniform(1.0, 4.0, 600), [1.0, 2.0, 4.0 - 2.0 ** -22, 1.0 + 2.0 ** -23]]).astype(np.float32):
        a = F(a32) * Fraction(4) ** int(rng.integers(-20, 30))
        root = F(np.sqrt(np.float64(float(a))))           # double: far closer than the decisions below need
        want = _rn32(root)
        assert (want - ulp(want) / 2) ** 2 < a < (want + ulp(want) / 2) ** 2 or want ** 2 == a
        prv, nxt = (lambda v: v - ulp(v - ulp(v) / 2)), (lambda v: v + ulp(v))  # the neighbouring floats (bit pattern -1 / +1)
        for s in (prv(want), want, nxt(want)):
            off = float(s - want)
            dn, up = prv(s), nxt(s)
            r_dn, r_up = fma(-dn, s, a), fma(-up, s, a)
            r = dn if r_dn <= 0 else s
            r = up if r_up > 0 else r
            assert r == want, (float(a), off)


def test_banded_magnitude_table_counts_thresholds(oracle):
    """The fp32 encoder's magnitude code: entry floor(12.5 |u|) of a 16-entry table names the thresholds below its
    band of width 0.08, the one threshold inside and the centres either side; code = count + (threshold < |u|).
    Simulated in float32 (the index is floor(200 |u|) with its low four bits cleared, the product rounded as the
    GPU rounds it) against the plain count, on every float32 within 3000 ulp of a band edge or a threshold and on a
    random sample."""
    thr, cen = oracle.mag_constants()
    thr, cen = thr.astype(np.float32), cen.astype(np.float32)
    slop = 1e-4
    below, inside_thr, c_lo, c_hi = [], [], [], []
    for k in range(16):
        lo, hi = np.float32(k) / np.float32(12.5) - np.float32(slop), np.float32(k + 1) / np.float32(12.5) + np.float32(slop)
        b = int((thr <= lo).sum())
        ins = thr[(thr > lo) & (thr < hi)]
        assert ins.size <= 1, k
        below.append(b)
        inside_thr.append(ins[0] if ins.size else np.float32(np.inf))
        c_lo.append(cen[b])
        c_hi.append(cen[b + (1 if ins.size else 0)])
    below, inside_thr, c_lo, c_hi = map(np.asarray, (below, inside_thr, c_lo, c_hi))
    rng = np.random.default_rng(5)
    anchors = np.concatenate([np.arange(1, 14, dtype=np.float32) / np.float32(12.5), thr, [np.float32(1.0)]]).astype(np.float32)
    near = (anchors.view(np.uint32)[:, None] + np.arange(-3000, 3001)[None, :]).astype(np.uint32).view(np.float32).ravel()
    au = np.concatenate([near, rng.uniform(0, 1.0000005, 200000).astype(np.float32), np.float32([0.0, 1e-30, 1.0000001])])
    au = au[au <= np.float32(1.001)]
    idx = ((au * np.float32(200.0)).astype(np.float32).astype(np.uint32) & 0xF0) >> 4
    above = inside_thr[idx] < au
    code = below[idx] + above
    want = (thr[None, :] < au[:, None]).sum(axis=1)
    assert np.array_equal(code, want)
    assert np.array_equal(np.where(above, c_hi[idx], c_lo[idx]), cen[want])
