"""Pins the CPU oracle against what the mathematics fixes.

The reference holds no golden vectors for this path (its tests assert invariants
between two of its own GPU code paths), so every oracle function is pinned by a
closed form, an invariant, a brute force or a known-answer vector that a
plausible mistake (dropped term, wrong sign/index, transposed operand, wrong
stage order) would break.  The invariants themselves are the ones the reference
asserts: tests/test_core.py:15-109, tests/test_prerot.py:43-159,
tests/test_sparse_v.py:47-168, tests/test_flash_attention.py:38-137.
"""
import math

import numpy as np
import pytest

from oracle import polarquant_oracle as o

F32 = np.float32


def hadamard_dense(d):
    j = np.arange(d)
    pop = np.array([[bin(a & b).count("1") for b in j] for a in j])
    return np.where(pop % 2 == 0, 1.0, -1.0)


def sylvester(d):
    H = np.array([[1.0]])
    while H.shape[0] < d:
        H = np.block([[H, H], [H, -H]])
    return H


# ---------------------------------------------------------------- rotation

@pytest.mark.parametrize("d", [2, 8, 32, 64, 128, 256])
def test_butterfly_is_sylvester_hadamard(d):
    assert np.array_equal(hadamard_dense(d), sylvester(d))
    # integers below 2^24/d are exact in float32, so the butterfly must equal H @ x exactly
    rng = np.random.default_rng(d)
    x = rng.integers(-1000, 1000, size=(5, d)).astype(F32)
    assert np.array_equal(o.raw_butterfly(x), (x.astype(np.float64) @ hadamard_dense(d)).astype(F32))


def test_butterfly_stage_order_bitexact_vs_scalar_loop():
    # in-place scalar restatement of the loop at metal.py:51-64
    rng = np.random.default_rng(1)
    x = rng.standard_normal((3, 128)).astype(F32)
    ref = x.copy()
    for row in ref:
        h = 1
        while h < 128:
            for j in range(128):
                if (j // h) % 2 == 0:
                    a, b = row[j], row[j + h]
                    row[j], row[j + h] = F32(a + b), F32(a - b)
            h *= 2
    assert np.array_equal(o.raw_butterfly(x), ref)


def test_wht_involution_and_norm():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((8, 128)).astype(F32)
    y = o.walsh_hadamard_transform(x)
    assert np.abs(o.walsh_hadamard_transform(y) - x).max() < 1e-5      # test_core.py:15-24
    assert np.abs(np.linalg.norm(y, axis=-1) - np.linalg.norm(x, axis=-1)).max() < 1e-4
    s = o.random_diagonal_sign(128, 7)
    z = o.inverse_randomized_hadamard(o.randomized_hadamard_transform(x, s), s)
    assert np.abs(z - x).max() < 1e-4                                      # test_core.py:39-48
    assert o.wht_scale(128).view(np.uint32) == 0x3DB504F3


def test_wht_rejects_non_power_of_two():
    with pytest.raises(AssertionError):
        o.raw_butterfly(np.zeros((1, 96), F32))


def test_signs_are_pm1_and_seeded():
    a = o.random_diagonal_sign(128, 42)
    assert set(np.unique(a)) <= {-1.0, 1.0} and a.dtype == F32
    assert np.array_equal(a, o.random_diagonal_sign(128, 42))
    assert not np.array_equal(a, o.random_diagonal_sign(128, 43))
    assert 40 < (a > 0).sum() < 88
    assert a[:8].tolist() == [-1, 1, -1, -1, 1, 1, 1, 1]                # frozen generator


def test_kurtosis_after_rotation():
    # test_core.py:51-67: a spiky vector becomes near-Gaussian after the rotation
    rng = np.random.default_rng(3)
    x = np.zeros((64, 256), F32)
    x[:, :4] = rng.standard_normal((64, 4)) * 10
    y = o.randomized_hadamard_transform(x, o.random_diagonal_sign(256, 42))
    k = ((y - y.mean()) ** 4).mean() / (y.var() ** 2)
    assert 1.5 < k < 6.0


# ---------------------------------------------------------------- codebook

def test_boundaries_hex():
    b = o.gaussian_boundaries(o.gaussian_codebook(3)).view(np.uint32)
    assert [hex(v) for v in b] == ["0xbfdfbe76", "0xbf866666", "0xbf00240b", "0x0",
                                   "0x3f00240b", "0x3f866666", "0x3fdfbe76"]
    for bits in (1, 2, 3, 4):
        c = o.gaussian_codebook(bits)
        assert len(c) == 2 ** bits and np.array_equal(c, -c[::-1])
    with pytest.raises(ValueError):
        o.gaussian_codebook(5)


# ---------------------------------------------------------------- packing

@pytest.mark.parametrize("bits", [1, 2, 3, 4])
def test_pack_exhaustive_slots(bits):
    vpw = o.VALS_PER_WORD[bits]
    dim = 128
    pd = o.packed_dim(dim, bits)
    assert pd == -(-dim // vpw)
    for e in (0, 1, vpw - 1, vpw, dim - 1):
        for v in range(2 ** bits):
            idx = np.zeros((1, dim), np.uint8)
            idx[0, e] = v
            p = o.pack_indices(idx, bits)
            want = np.zeros(pd, np.uint64)
            want[e // vpw] = v << ((e % vpw) * bits)
            assert np.array_equal(p[0].astype(np.uint64), want)
    rng = np.random.default_rng(bits)
    idx = rng.integers(0, 2 ** bits, size=(3, 5, dim)).astype(np.uint8)
    p = o.pack_indices(idx, bits)
    assert p.shape == (3, 5, pd) and p.dtype == np.uint32
    assert np.array_equal(o.unpack_indices(p, bits, dim), idx)


def test_pack_3bit_layout_d128():
    idx = np.full((1, 128), 7, np.uint8)
    p = o.pack_indices(idx, 3)[0]
    assert p.shape == (13,)
    assert all(int(w) == 0x3FFFFFFF for w in p[:12]) and int(p[12]) == 0x00FFFFFF
    assert o.packed_dim(128, 3) == 13 and o.packed_dim(64, 4) == 8 and o.packed_dim(32, 2) == 2


# ---------------------------------------------------------------- quantize

def _q3(x, signs=None, variant="mlx"):
    d = x.shape[-1]
    signs = np.ones(d, F32) if signs is None else signs
    b = o.gaussian_boundaries(o.gaussian_codebook(3))
    return o.quantize(x, signs, b, variant)


def test_quantize_kat_zero_vector():
    p, n = o.fused_quantize(np.zeros((2, 128), np.float16), np.ones(128, F32),
                            o.gaussian_boundaries(o.gaussian_codebook(3)), 128, 3)
    assert n.tolist() == [0.0, 0.0]
    assert [int(w) for w in p[0]] == [0x1B6DB6DB] * 12 + [0x006DB6DB]


@pytest.mark.parametrize("variant", ["mlx", "metal"])
def test_quantize_kat_one_hot(variant):
    for j, a in ((5, 3.0), (0, 0.25), (127, 1000.0)):
        x = np.zeros((1, 128), F32)
        x[0, j] = a
        idx, n = _q3(x, variant=variant)
        assert n[0] == F32(a)
        want = np.array([5 if bin(j & k).count("1") % 2 == 0 else 2 for k in range(128)], np.uint8)
        assert np.array_equal(idx[0], want)
    x = np.zeros((1, 128), F32)
    x[0, 5] = 3.0
    p = o.pack_indices(_q3(x)[0], 3)[0]
    assert [int(w) for w in p[:3]] == [0x15AAA555, 0x1556AA95, 0x2A555AAA]


def test_quantize_invariants():
    rng = np.random.default_rng(4)
    x = rng.standard_normal((256, 128)).astype(np.float16)
    s = o.random_diagonal_sign(128, 43)
    idx, n = _q3(x, s)
    # power-of-two scaling is exact in float32: indices identical, norms scale
    idx2, n2 = _q3(x.astype(F32) * F32(4.0), s)
    assert np.array_equal(idx, idx2) and np.array_equal(n2, n * F32(4.0))
    # negation mirrors the symmetric codebook (no value sits exactly on a boundary here)
    idx3, _ = _q3(-x.astype(F32), s)
    assert np.array_equal(idx3, 7 - idx)
    # norms: tree order equals the float64 norm to float32 accuracy
    ref = np.linalg.norm(x.astype(np.float64), axis=-1)
    assert np.abs(n - ref).max() < 2e-6 * ref.max()


def test_quantize_is_nearest_centroid_bruteforce():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((64, 128)).astype(F32)
    s = o.random_diagonal_sign(128, 42)
    c = o.gaussian_codebook(3)
    idx, n = _q3(x, s, "metal")
    z = o.raw_butterfly((x / n[:, None]) * s).astype(np.float64)
    brute = np.abs(z[..., None] - c.astype(np.float64)).argmin(-1)
    assert np.array_equal(idx, brute.astype(np.uint8))


def test_quantize_tie_nan_and_strictness():
    b = o.gaussian_boundaries(o.gaussian_codebook(3))
    # a value exactly on a boundary stays in the lower bin (strict >, quantizer.py:104)
    z = np.array([b[4], np.nextafter(b[4], F32(9), dtype=F32)], F32)
    got = [(z[i] > b).sum() for i in range(2)]
    assert got == [4, 5]
    x = np.full((1, 128), np.nan, F32)
    idx, _ = _q3(x)
    assert (idx == 0).all()


def test_quantize_variants_differ_only_in_double_rounding():
    rng = np.random.default_rng(6)
    x = rng.standard_normal((512, 128)).astype(np.float16)
    s = o.random_diagonal_sign(128, 43)
    i1, n1 = _q3(x, s, "mlx")
    i2, n2 = _q3(x, s, "metal")
    assert np.array_equal(n1, n2)
    assert (i1 != i2).mean() < 1e-4


def test_config1_statistics():
    # benchmark configuration 1: [1,4,1024,128] fp16 N(0,1); textbook 8-level Lloyd-Max distortion
    rng = np.random.default_rng(0)
    x = rng.standard_normal((1, 4, 1024, 128)).astype(np.float16)
    s = o.random_diagonal_sign(128, 43)
    c = o.gaussian_codebook(3)
    idx, n = o.quantize(x, s, o.gaussian_boundaries(c))
    assert idx.shape == (1, 4, 1024, 128) and n.shape == (1, 4, 1024)
    xh = o.dequantize(idx, n, c, s)
    x32 = x.astype(F32)
    mse = float(((xh - x32) ** 2).mean())
    cos = float((np.sum(xh * x32, -1) / np.linalg.norm(xh, axis=-1) / np.linalg.norm(x32, axis=-1)).mean())
    assert 0.032 < mse < 0.036 and 0.981 < cos < 0.985
    hist = np.bincount(idx.ravel(), minlength=8) / idx.size
    assert np.abs(hist - [.040, .108, .162, .191, .190, .161, .108, .040]).max() < 0.004


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_roundtrip_quality_ordering(bits):
    rng = np.random.default_rng(7)                                        # test_core.py:70-109
    x = rng.standard_normal((128, 128)).astype(F32)
    s = o.random_diagonal_sign(128, 42)
    c = o.gaussian_codebook(bits)
    idx, n = o.quantize(x, s, o.gaussian_boundaries(c))
    xh = o.dequantize(idx, n, c, s)
    cos = (np.sum(xh * x, -1) / np.linalg.norm(xh, axis=-1) / np.linalg.norm(x, axis=-1)).mean()
    assert cos > {2: 0.90, 3: 0.97, 4: 0.99}[bits]


# ---------------------------------------------------------------- dequant / scores

def test_dequant_matches_dense_hadamard_f64():
    rng = np.random.default_rng(8)
    for d, bits in ((128, 3), (64, 4), (32, 2)):
        c = o.gaussian_codebook(bits)
        s = o.random_diagonal_sign(d, 42)
        idx = rng.integers(0, 2 ** bits, size=(17, d)).astype(np.uint8)
        n = (rng.random(17) * 10 + 0.1).astype(F32)
        want = (c.astype(np.float64)[idx] @ hadamard_dense(d)) * s / d * n[:, None]
        got = o.packed_dequantize(o.pack_indices(idx, bits), n, c, s, d, bits)
        assert np.abs(got - want).max() < 2e-6 * np.abs(want).max()
        assert o.dequant_fp16(o.pack_indices(idx, bits), n, c, s, d, bits).dtype == np.float16


def test_prerotate_is_raw_butterfly_of_signed_q():
    rng = np.random.default_rng(9)
    q = rng.standard_normal((4, 128)).astype(F32)
    s = o.random_diagonal_sign(128, 1)
    want = (q * s).astype(np.float64) @ hadamard_dense(128)
    assert np.allclose(o.prerotate_query(q, s), want, atol=1e-4)         # test_prerot.py:43-59
    with pytest.raises(ValueError):
        o.prerotate_query(q[0], s)


@pytest.mark.parametrize("H,S,D,bits", [(4, 64, 128, 3), (8, 256, 128, 3), (2, 16, 64, 4), (1, 128, 32, 2)])
def test_prerot_scores_equal_dot_with_dequant(H, S, D, bits):
    rng = np.random.default_rng(10)                                       # test_prerot.py:62-97
    c = o.gaussian_codebook(bits)
    s = o.random_diagonal_sign(D, 42)
    kp = o.pack_indices(rng.integers(0, 2 ** bits, size=(H, S, D)).astype(np.uint8), bits)
    kn = (rng.random((H, S)) * 10 + 1).astype(F32)
    q = rng.standard_normal((H, D)).astype(F32)
    full = o.packed_fused_qk_scores(q, kp, kn, c, s, D, bits)
    pre = o.prerot_fused_qk_scores(o.prerotate_query(q, s), kp, kn, c, D, bits)
    assert np.abs(full - pre).max() < 1e-4 * max(1.0, np.abs(full).max())


@pytest.mark.parametrize("n_kv,n_rep", [(4, 2), (2, 4), (4, 7)])
def test_prerot_scores_gqa_equals_repeat(n_kv, n_rep):
    rng = np.random.default_rng(11)                                       # test_prerot.py:100-133
    D, S, bits = 128, 48, 3
    c = o.gaussian_codebook(bits)
    kp = o.pack_indices(rng.integers(0, 8, size=(n_kv, S, D)).astype(np.uint8), bits)
    kn = (rng.random((n_kv, S)) + 0.5).astype(F32)
    qr = rng.standard_normal((n_kv * n_rep, D)).astype(F32)
    a = o.prerot_fused_qk_scores(qr, kp, kn, c, D, bits, n_rep)
    b = o.prerot_fused_qk_scores(qr, np.repeat(kp, n_rep, 0), np.repeat(kn, n_rep, 0), c, D, bits, 1)
    assert np.array_equal(a, b)
    with pytest.raises(ValueError, match="must equal n_kv_heads"):
        o.prerot_fused_qk_scores(qr[:-1], kp, kn, c, D, bits, n_rep)


# ---------------------------------------------------------------- sparse V / flash

def _v_fixture(rng, n_kv, S, D, bits):
    c = o.gaussian_codebook(bits)
    s = o.random_diagonal_sign(D, 43)
    vp = o.pack_indices(rng.integers(0, 2 ** bits, size=(n_kv, S, D)).astype(np.uint8), bits)
    vn = (rng.random((n_kv, S)) + 0.1).astype(F32)
    return c, s, vp, vn


def _softmax(x):
    e = np.exp(x - x.max(-1, keepdims=True))
    return (e / e.sum(-1, keepdims=True)).astype(F32)


@pytest.mark.parametrize("H,S,D,bits", [(4, 128, 128, 3), (2, 512, 128, 3), (8, 64, 64, 4)])
def test_sparse_v_threshold_zero_is_dense(H, S, D, bits):
    rng = np.random.default_rng(12)                                       # test_sparse_v.py:47-76
    c, s, vp, vn = _v_fixture(rng, H, S, D, bits)
    w = _softmax(rng.standard_normal((H, S)) * 3)
    vd = o.packed_dequantize(vp.reshape(H * S, -1), vn.reshape(-1), c, s, D, bits).reshape(H, S, D)
    want = np.einsum("hs,hsd->hd", w.astype(np.float64), vd.astype(np.float64))
    got = o.sparse_v_matvec(w, vp, vn, c, s, D, bits, threshold=0.0)
    assert np.abs(got - want).max() / np.abs(want).max() < 1e-5


def test_sparse_v_threshold_semantics():
    rng = np.random.default_rng(13)
    H, S, D, bits = 4, 256, 128, 3
    c, s, vp, vn = _v_fixture(rng, H, S, D, bits)
    w = _softmax(rng.standard_normal((H, S)) * 5)
    dense = o.sparse_v_matvec(w, vp, vn, c, s, D, bits, threshold=0.0)
    # masking by hand on the final weights == the thresholded call (sparse_v.py:60-61)
    thr = 1e-3
    wm = np.where(w < F32(thr), F32(0), w)
    assert np.array_equal(o.sparse_v_matvec(w, vp, vn, c, s, D, bits, threshold=thr),
                          o.sparse_v_matvec(wm, vp, vn, c, s, D, bits, threshold=0.0))
    sp = o.sparse_v_matvec(w, vp, vn, c, s, D, bits, threshold=1e-5)
    cosv = (sp * dense).sum() / np.linalg.norm(sp) / np.linalg.norm(dense)
    assert cosv > 0.999                                                   # test_sparse_v.py:79-109
    # threshold above every weight -> exactly zero (test_sparse_v.py:150-168)
    z = o.sparse_v_matvec(w, vp, vn, c, s, D, bits, threshold=2.0)
    assert (z == 0).all()
    # negative threshold means dense (sparse_v.py:164)
    assert np.array_equal(o.sparse_v_matvec(w, vp, vn, c, s, D, bits, threshold=-1.0), dense)
    assert o.count_active_positions(w, 1e-5) == int((w > 1e-5).sum())


def test_sparse_v_gqa_and_errors():
    rng = np.random.default_rng(14)                                       # test_sparse_v.py:112-147
    n_kv, n_rep, S, D, bits = 4, 7, 96, 128, 3
    c, s, vp, vn = _v_fixture(rng, n_kv, S, D, bits)
    w = _softmax(rng.standard_normal((n_kv * n_rep, S)))
    a = o.sparse_v_matvec(w, vp, vn, c, s, D, bits, 0.0, n_rep)
    b = o.sparse_v_matvec(w, np.repeat(vp, n_rep, 0), np.repeat(vn, n_rep, 0), c, s, D, bits, 0.0, 1)
    assert np.abs(a - b).max() < 1e-6
    with pytest.raises(ValueError, match="power of 2"):
        o.sparse_v_matvec(w, vp, vn, c, s, 96, bits)
    with pytest.raises(ValueError, match="dim > 256"):
        o.sparse_v_matvec(w, vp, vn, c, s, 512, bits)
    with pytest.raises(ValueError, match="must equal n_kv_heads"):
        o.sparse_v_matvec(w[:-1], vp, vn, c, s, D, bits, 0.0, n_rep)


@pytest.mark.parametrize("n_kv,n_rep,S", [(4, 1, 96), (2, 4, 200), (4, 7, 64)])
def test_flash_equals_dense_attention_on_dequantised_kv(n_kv, n_rep, S):
    rng = np.random.default_rng(15)                                       # test_flash_attention.py:38-137
    D, bits = 128, 3
    c = o.gaussian_codebook(bits)
    ks, vs = o.random_diagonal_sign(D, 42), o.random_diagonal_sign(D, 43)
    b = o.gaussian_boundaries(c)
    K = rng.standard_normal((n_kv, S, D)).astype(np.float16)
    V = rng.standard_normal((n_kv, S, D)).astype(np.float16)
    kp, kn = o.fused_quantize(K.reshape(-1, D), ks, b, D, bits)
    vp, vn = o.fused_quantize(V.reshape(-1, D), vs, b, D, bits)
    kp, kn, vp, vn = kp.reshape(n_kv, S, -1), kn.reshape(n_kv, S), vp.reshape(n_kv, S, -1), vn.reshape(n_kv, S)
    q = rng.standard_normal((n_kv * n_rep, D)).astype(F32)
    sc = 1 / math.sqrt(D)
    got = o.flash_attention_turboquant(o.prerotate_query(q, ks), kp, kn, vp, vn, c, c, vs, D, bits, sc, 16, n_rep)
    kd = o.packed_dequantize(kp.reshape(-1, 13), kn.reshape(-1), c, ks, D, bits).reshape(n_kv, S, D)
    vd = o.packed_dequantize(vp.reshape(-1, 13), vn.reshape(-1), c, vs, D, bits).reshape(n_kv, S, D)
    want = o.dense_attention(q[:, None, :], kd, vd, sc)[:, 0, :]
    assert np.abs(got - want).max() < 1e-5 * max(1, np.abs(want).max()) + 1e-5
    comp = o.turboquant_attention_single(q, kp, kn, vp, vn, c, ks, c, vs, D, bits, sc)
    assert np.abs(got - comp).max() < 1e-5
    with pytest.raises(ValueError, match="block_size"):
        o.flash_attention_turboquant(q, kp, kn, vp, vn, c, c, vs, D, bits, sc, 33, n_rep)
    with pytest.raises(ValueError, match="<= 128"):
        o.flash_attention_turboquant(q, kp, kn, vp, vn, c, c, vs, 256, bits, sc, 16, n_rep)


def test_vonly_decode_equals_dense_attention():
    rng = np.random.default_rng(16)
    n_kv, n_rep, S, D, bits = 4, 7, 300, 128, 3
    c = o.gaussian_codebook(bits)
    vs = o.random_diagonal_sign(D, 43)
    K = rng.standard_normal((n_kv, S, D)).astype(np.float16)
    V = rng.standard_normal((n_kv, S, D)).astype(np.float16)
    vp, vn = o.fused_quantize(V.reshape(-1, D), vs, o.gaussian_boundaries(c), D, bits)
    vp, vn = vp.reshape(n_kv, S, -1), vn.reshape(n_kv, S)
    q = rng.standard_normal((n_kv * n_rep, D)).astype(np.float16)
    sc = 1 / math.sqrt(D)
    got = o.vonly_decode_attention(q, K, vp, vn, c, vs, D, bits, sc)
    vd = o.packed_dequantize(vp.reshape(-1, 13), vn.reshape(-1), c, vs, D, bits).reshape(n_kv, S, D)
    want = o.dense_attention(q.astype(np.float64)[:, None, :], K, vd, sc)[:, 0, :]
    assert np.abs(got - want).max() < 1e-5
    # quantised V stays close to fp16 V attention: cosine > 0.95 on the output
    full = o.dense_attention(q.astype(np.float64)[:, None, :], K, V, sc)[:, 0, :]
    cosv = (got * full).sum() / np.linalg.norm(got) / np.linalg.norm(full)
    assert cosv > 0.95


def test_prefill_attention_rows_are_prefix_flash_decodes():
    """Pins the causal indexing of prefill_attention: row i of a chunk that starts at q_pos0 must be
    the single-token flash attention (rotated-domain formula, pinned above) over positions
    0 .. q_pos0 + i; and without the causal rule every row sees all positions."""
    rng = np.random.default_rng(77)
    n_kv, n_rep, T, D, bits, n_rows, pos0 = 2, 2, 50, 128, 3, 7, 43
    c = o.gaussian_codebook(bits)
    b = o.gaussian_boundaries(c)
    ks, vs = o.random_diagonal_sign(D, 42), o.random_diagonal_sign(D, 43)
    K = rng.standard_normal((n_kv * T, D)).astype(np.float16)
    V = rng.standard_normal((n_kv * T, D)).astype(np.float16)
    kp, kn = o.fused_quantize(K, ks, b, D, bits)
    vp, vn = o.fused_quantize(V, vs, b, D, bits)
    kp, vp = kp.reshape(n_kv, T, -1), vp.reshape(n_kv, T, -1)
    kn, vn = kn.reshape(n_kv, T), vn.reshape(n_kv, T)
    q = rng.standard_normal((n_kv * n_rep, n_rows, D)).astype(np.float32)
    sc = 1 / np.sqrt(D)
    got = o.prefill_attention(q, kp, kn, vp, vn, c, c, ks, vs, D, bits, sc, pos0, n_rep)
    assert got.shape == (n_kv * n_rep, n_rows, D)
    for i in (0, 3, n_rows - 1):
        L = pos0 + i + 1
        want = o.flash_attention_turboquant(o.prerotate_query(q[:, i], ks), kp[:, :L], kn[:, :L], vp[:, :L],
                                            vn[:, :L], c, c, vs, D, bits, sc, 16, n_rep)
        assert np.allclose(got[:, i], want, rtol=1e-5, atol=1e-6)
    full = o.prefill_attention(q, kp, kn, vp, vn, c, c, ks, vs, D, bits, sc, pos0, n_rep, causal=False)
    want = o.flash_attention_turboquant(o.prerotate_query(q[:, 2], ks), kp, kn, vp, vn, c, c, vs, D, bits, sc, 16, n_rep)
    assert np.allclose(full[:, 2], want, rtol=1e-5, atol=1e-6)


# ------------------------------------------------------------------ committed closed-form vectors

def _golden_cases():
    import json
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "kat_vectors.json")
    with open(path) as f:
        return json.load(f)["cases"]


@pytest.mark.parametrize("case", _golden_cases(), ids=lambda c: c["name"])
@pytest.mark.parametrize("variant", ["mlx", "metal"])
def test_oracle_reproduces_closed_form_vectors(case, variant):
    """tests/golden/kat_vectors.json is derived in exact rational arithmetic from the Hadamard closed
    form (tests/golden/make_kat_vectors.py, no oracle code involved): indices, packed words and norms
    must match bit for bit, the dequantised vector to float32 rounding."""
    d, bits = case["dim"], case["bits"]
    x = np.array(case["x"], np.float32)[None, :]
    s = np.array(case["signs"], np.float32)
    c = o.gaussian_codebook(bits)
    b = o.gaussian_boundaries(c)
    idx, nrm = o.quantize(x, s, b, variant)
    assert idx[0].tolist() == case["idx"]
    assert float(nrm.reshape(-1)[0]) == case["norm"]
    want_words = np.array([int(w, 16) for w in case["packed_hex"]], np.uint32)
    assert np.array_equal(o.pack_indices(idx, bits)[0], want_words)
    p, n = o.fused_quantize(x, s, b, d, bits, variant)
    assert np.array_equal(p[0], want_words) and float(n[0]) == case["norm"]
    deq = o.packed_dequantize(p, n, c, s, d, bits)[0].astype(np.float64)
    want = np.array(case["dequant"])
    assert np.abs(deq - want).max() <= 2e-6 * max(1.0, np.abs(want).max())
