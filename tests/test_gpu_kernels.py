"""GPU parity tests: every HIP kernel, called through the C-ABI library, against the CPU oracle
on the same seeded inputs.  Integer outputs (packed indices) must be bit-exact; float outputs are
held to the tolerance written in each test.  Cases mirror the reference's own test parameters
(tests/test_prerot.py, tests/test_sparse_v.py, tests/test_flash_attention.py, tests/test_core.py).
"""
import math

import numpy as np
import pytest

torch = pytest.importorskip("torch")

from oracle import polarquant_oracle as o  # noqa: E402

pytestmark = pytest.mark.gpu

F32 = np.float32
REL, ABS = 2e-3, 1e-3          # attention-output tolerance of the task statement


@pytest.fixture(scope="module")
def tq():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a GPU: torch.cuda.is_available() is False")
    import tqhip
    return tqhip


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def tables(bits):
    c = o.gaussian_codebook(bits)
    return c, o.gaussian_boundaries(c)


def close(got, want, rel=REL, abs_=ABS, row_scale=False, extra=0.0):
    """|err| <= abs + rel * |want| elementwise; with row_scale the relative part is taken against the
    largest magnitude of the output row (the reference's own measure, tests/test_flash_attention.py:
    max_abs / max_ref), which is the meaningful one when an outlier channel dominates a row: the
    Hadamard mixing spreads any operand rounding over all elements of the row."""
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    ref = np.abs(want).max(axis=-1, keepdims=True) if row_scale else np.abs(want)
    ok = err <= abs_ + rel * ref + extra
    assert ok.all(), f"max err {err.max():.3e} (want scale {np.abs(want).max():.3e}), {(~ok).sum()} bad"


def threshold_slack(w, thr, vp, vn, c, vs, n_rep, band):
    """Extra tolerance for a thresholded value sum over PACKED keys (the only users): the scores of that step come
    from fp16 operands (about 3e-4 relative per score, i.e. up to ~2e-3 relative per weight at |score| ~ 6), so a
    weight within `band` (relative; 3e-3 in the tests) of the threshold may fall on either side of it; such a
    position moves the output by its whole contribution w * |dequantised V row|.  Returns (n_q, dim): the sum of
    those contributions over the ambiguous positions of each head -- zero when no weight is that close, in which
    case the plain 2e-3 / 1e-3 bar applies.  The thresholded steps over fp16 keys do not use it."""
    amb = np.abs(w.astype(np.float64) - thr) <= band * thr                      # (n_q, T)
    if not amb.any():
        return np.zeros((w.shape[0], 128))
    n_kv, T = vn.shape
    vhat = np.abs(o.packed_dequantize(vp.reshape(-1, vp.shape[-1]), vn.reshape(-1), c, vs, 128, 3)).reshape(n_kv, T, 128)
    wa = (w * amb).reshape(n_kv, n_rep, T).astype(np.float64)
    return np.matmul(wa, vhat.astype(np.float64)).reshape(-1, 128)


# ------------------------------------------------------------------ encode

@pytest.mark.parametrize("variant", ["mlx", "metal"])
@pytest.mark.parametrize("dim,bits", [(128, 3), (128, 4), (128, 2), (128, 1), (64, 4), (64, 3), (32, 2),
                                      (32, 3), (256, 3), (256, 4)])
def test_encode_bit_exact(tq, dim, bits, variant):
    rng = np.random.default_rng(dim * 10 + bits)
    x = rng.standard_normal((1037, dim)).astype(np.float16)       # ragged count: not a multiple of 4
    s = o.random_diagonal_sign(dim, 43)
    c, b = tables(bits)
    wp, wn = o.fused_quantize(x, s, b, dim, bits, variant)
    gp, gn = tq.fused_quantize(dev(x), dev(s), b, dim, bits, variant=variant)
    assert gp.dtype == torch.uint32 and gp.shape == wp.shape
    assert np.array_equal(host(gp), wp)
    assert np.array_equal(host(gn), wn)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_encode_dtypes_and_scales(tq, dtype):
    rng = np.random.default_rng(1)
    x = (rng.standard_normal((513, 128)) * rng.choice([1e-3, 1.0, 300.0], size=(513, 1))).astype(dtype)
    s = o.random_diagonal_sign(128, 42)
    c, b = tables(3)
    wp, wn = o.fused_quantize(x, s, b, 128, 3)
    gp, gn = tq.fused_quantize(dev(x), dev(s), b, 128, 3)
    assert np.array_equal(host(gp), wp) and np.array_equal(host(gn), wn)


def test_encode_bf16_input(tq):
    rng = np.random.default_rng(2)
    xt = torch.from_numpy(rng.standard_normal((200, 128)).astype(F32)).to(torch.bfloat16)
    s = o.random_diagonal_sign(128, 42)
    c, b = tables(3)
    wp, wn = o.fused_quantize(xt.float().numpy(), s, b, 128, 3)
    gp, gn = tq.fused_quantize(xt.cuda(), dev(s), b, 128, 3)
    assert np.array_equal(host(gp), wp) and np.array_equal(host(gn), wn)


def test_encode_known_answers(tq):
    c, b = tables(3)
    ones = np.ones(128, F32)
    x = np.zeros((3, 128), np.float16)
    x[1, 5] = 3.0
    x[2, :] = np.nan
    gp, gn = tq.fused_quantize(dev(x), dev(ones), b, 128, 3)
    gp, gn = host(gp), host(gn)
    assert [int(w) for w in gp[0]] == [0x1B6DB6DB] * 12 + [0x006DB6DB] and gn[0] == 0.0
    assert [int(w) for w in gp[1][:3]] == [0x15AAA555, 0x1556AA95, 0x2A555AAA] and gn[1] == 3.0
    assert (gp[2] == 0).all() and np.isnan(gn[2])
    # empty input
    ep, en = tq.fused_quantize(torch.zeros((0, 128), dtype=torch.float16, device="cuda"), dev(ones), b, 128, 3)
    assert ep.shape == (0, 13) and en.shape == (0,)


def test_encode_near_boundary_values(tq):
    """Vectors built so that butterfly outputs sit within a few ulp of decision boundaries: the
    double-rounding rule of the pure-array quantiser and the raw rule of the Metal encoder must
    each be reproduced exactly."""
    c, b = tables(3)
    ones = np.ones(128, F32)
    rng = np.random.default_rng(3)
    rows = []
    H = np.array([[1.0 if bin(j & k).count("1") % 2 == 0 else -1.0 for k in range(128)] for j in range(128)])
    for _ in range(400):
        z = rng.standard_normal(128)
        k = rng.integers(0, 128)
        z[k] = float(b[rng.integers(0, 7)]) * (1 + rng.integers(-3, 4) * 2.0 ** -23)
        z *= math.sqrt(128) / np.linalg.norm(z)
        rows.append((H @ z) / 128.0)
    x = np.array(rows, dtype=F32)
    for variant in ("mlx", "metal"):
        wp, wn = o.fused_quantize(x, ones, b, 128, 3, variant)
        gp, gn = tq.fused_quantize(dev(x), dev(ones), b, 128, 3, variant=variant)
        assert np.array_equal(host(gp), wp) and np.array_equal(host(gn), wn)


def test_config1_roundtrip(tq):
    """benchmark configuration 1: [1,4,1024,128] fp16 N(0,1): indices bit-exact, reconstruction MSE equal."""
    rng = np.random.default_rng(0)
    x = rng.standard_normal((1, 4, 1024, 128)).astype(np.float16)
    s = o.random_diagonal_sign(128, 43)
    c, b = tables(3)
    wp, wn = o.fused_quantize(x.reshape(-1, 128), s, b, 128, 3)
    gp, gn = tq.fused_quantize(dev(x.reshape(-1, 128)), dev(s), b, 128, 3)
    assert np.array_equal(host(gp), wp) and np.array_equal(host(gn), wn)
    wd = o.packed_dequantize(wp, wn, c, s, 128, 3)
    gd = host(tq.packed_dequantize(gp, gn, c, dev(s), 128, 3))
    assert np.array_equal(gd, wd)
    x32 = x.reshape(-1, 128).astype(F32)
    assert abs(float(((gd - x32) ** 2).mean()) - float(((wd - x32) ** 2).mean())) == 0.0
    assert 0.032 < float(((gd - x32) ** 2).mean()) < 0.036
    # fp16 norms, as the config text allows: a cast of the float32 norms
    assert np.array_equal(host(gn.to(torch.float16)), wn.astype(np.float16))


def _special_rows(rng, n, b):
    """n x 128 float32 rows: random scales, a zero row, one-hot rows, and rows whose butterfly
    outputs sit within a few ulp of a decision boundary."""
    x = (rng.standard_normal((n, 128)) * rng.choice([1e-3, 1.0, 300.0], size=(n, 1))).astype(F32)
    x[5] = 0.0
    x[6] = 0.0
    x[6, 127] = -2.5
    x[7] = 0.0
    x[7, 64] = 1e-3
    H = np.array([[1.0 if bin(j & k).count("1") % 2 == 0 else -1.0 for k in range(128)] for j in range(128)])
    for r in range(32, 232):
        z = rng.standard_normal(128)
        z[rng.integers(0, 128)] = float(b[rng.integers(0, 7)]) * (1 + rng.integers(-3, 4) * 2.0 ** -23)
        z *= math.sqrt(128) / np.linalg.norm(z)
        x[r] = (H @ z) / 128.0
    return x


@pytest.mark.parametrize("variant", ["mlx", "metal"])
@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_encode_streaming_kernel(tq, dtype, variant):
    """At d = 128 / 3-bit a row count that is a multiple of 16 takes the streaming encoder (four
    lanes per vector, reciprocal + fma division, guessed level + one compare): its bits must be the
    oracle's, for every input type and both threshold rules, special rows included."""
    rng = np.random.default_rng(31)
    c, b = tables(3)
    s = o.random_diagonal_sign(128, 43)
    n = 16 * 261
    x = _special_rows(rng, n, b)
    if dtype == "f32":
        xt = torch.from_numpy(x)
    elif dtype == "f16":
        xt = torch.from_numpy(x).to(torch.float16)
    else:
        xt = torch.from_numpy(x).to(torch.bfloat16)
    xt[100] = float("nan")
    xt[101, 3] = float("nan")
    ref_in = xt.float().numpy()
    ok = ~np.isnan(ref_in).any(axis=1)
    wp, wn = o.fused_quantize(ref_in[ok], s, b, 128, 3, variant)
    gp, gn = tq.fused_quantize(xt.cuda(), dev(s), b, 128, 3, variant=variant)
    gp, gn = host(gp), host(gn)
    assert np.array_equal(gp[ok], wp) and np.array_equal(gn[ok], wn)
    assert (gp[~ok] == 0).all() and np.isnan(gn[~ok]).all()          # NaN compares false with every threshold
    # the generic one-wavefront-per-vector kernel (ragged count) gives the same words
    gp2, gn2 = tq.fused_quantize(xt[: n - 3].cuda(), dev(s), b, 128, 3, variant=variant)
    assert np.array_equal(host(gp2), gp[: n - 3])
    assert np.array_equal(host(gn2)[ok[: n - 3]], gn[: n - 3][ok[: n - 3]])


def test_encode_and_dequant_into_strided_groups(tq):
    """Cache layout: groups (batch x head) of rows with a stride larger than the rows written, at a
    row offset; both streaming kernels must place every row where the generic ones do."""
    rng = np.random.default_rng(32)
    c, b = tables(3)
    s = o.random_diagonal_sign(128, 42)
    G, R, alloc, off = 3, 48, 256, 32
    x = rng.standard_normal((G, R, 128)).astype(np.float16)
    packed = torch.zeros((G, alloc, 13), dtype=torch.int32, device="cuda").view(torch.uint32)
    norms = torch.zeros((G, alloc), dtype=torch.float32, device="cuda")
    tq.encode_into(dev(x), dev(s), b, packed, norms, n_groups=G, rows_per_group=R, packed_group_stride=alloc,
                   norms_group_stride=alloc, dim=128, bits=3, packed_row_offset=off, norms_row_offset=off)
    wp, wn = o.fused_quantize(x.reshape(-1, 128), s, b, 128, 3)
    hp, hn = host(packed), host(norms)
    assert np.array_equal(hp[:, off:off + R], wp.reshape(G, R, 13)) and np.array_equal(hn[:, off:off + R], wn.reshape(G, R))
    assert (hp[:, :off] == 0).all() and (hp[:, off + R:] == 0).all() and (hn[:, off + R:] == 0).all()
    for dt in (torch.float32, torch.float16, torch.bfloat16):
        out = torch.zeros((G, alloc, 128), dtype=dt, device="cuda")
        tq.dequant_into(packed, norms, c, dev(s), out, n_groups=G, rows_per_group=R, packed_group_stride=alloc,
                        norms_group_stride=alloc, out_group_stride=alloc, dim=128, bits=3, packed_row_offset=off,
                        norms_row_offset=off, out_row_offset=off)
        want = torch.from_numpy(o.packed_dequantize(wp, wn, c, s, 128, 3)).to(dt).reshape(G, R, 128)
        assert torch.equal(out[:, off:off + R].cpu(), want)
        assert (out[:, :off] == 0).all() and (out[:, off + R:] == 0).all()


@pytest.mark.parametrize("dt", [torch.float32, torch.float16, torch.bfloat16])
def test_dequant_streaming_kernel(tq, dt):
    rng = np.random.default_rng(33)
    c, b = tables(3)
    s = o.random_diagonal_sign(128, 43)
    n = 16 * 70
    p = o.pack_indices(rng.integers(0, 8, size=(n, 128)).astype(np.uint8), 3)
    nr = (rng.random(n) * rng.choice([1e-3, 1.0, 500.0], size=n)).astype(F32)
    nr[3] = 0.0
    want = torch.from_numpy(o.packed_dequantize(p, nr, c, s, 128, 3)).to(dt)
    out = torch.empty((n, 128), dtype=dt, device="cuda")
    tq.dequant_into(dev(p), dev(nr), c, dev(s), out, n_groups=1, rows_per_group=n, packed_group_stride=n,
                    norms_group_stride=n, out_group_stride=n, dim=128, bits=3)
    assert torch.equal(out.cpu(), want)


# ------------------------------------------------------------------ dequant / prerotate

@pytest.mark.parametrize("dim,bits", [(128, 3), (64, 4), (32, 2), (256, 3), (128, 1)])
def test_dequant_bit_exact(tq, dim, bits):
    rng = np.random.default_rng(4)
    c, b = tables(bits)
    s = o.random_diagonal_sign(dim, 42)
    p = o.pack_indices(rng.integers(0, 2 ** bits, size=(333, dim)).astype(np.uint8), bits)
    n = (rng.random(333) * 10 + 0.1).astype(F32)
    want = o.packed_dequantize(p, n, c, s, dim, bits)
    got = host(tq.packed_dequantize(dev(p), dev(n), c, dev(s), dim, bits))
    assert got.dtype == F32 and np.array_equal(got, want)
    got16 = host(tq.dequant_fp16(dev(p), dev(n), c, dev(s), dim, bits))
    assert got16.dtype == np.float16 and np.array_equal(got16, want.astype(np.float16))


@pytest.mark.parametrize("dim", [32, 64, 128, 256])
def test_prerotate_query_bit_exact(tq, dim):
    rng = np.random.default_rng(5)
    q = rng.standard_normal((28, dim)).astype(F32)
    s = o.random_diagonal_sign(dim, 1)
    want = o.prerotate_query(q, s)
    assert np.array_equal(host(tq.prerotate_query(dev(q), dev(s))), want)
    q16 = q.astype(np.float16)
    assert np.array_equal(host(tq.prerotate_query(dev(q16), dev(s))), o.prerotate_query(q16, s))
    with pytest.raises(ValueError, match="expects"):
        tq.prerotate_query(dev(q[0]), dev(s))


def test_rotation_helpers(tq):
    rng = np.random.default_rng(6)
    x = rng.standard_normal((8, 128)).astype(F32)
    s = o.random_diagonal_sign(128, 42)
    assert np.array_equal(host(tq.random_diagonal_sign(128, 42, device="cuda")), s)
    y = tq.walsh_hadamard_transform(dev(x))
    assert np.array_equal(host(y), o.walsh_hadamard_transform(x))
    assert np.abs(host(tq.walsh_hadamard_transform(y)) - x).max() < 1e-5
    z = tq.inverse_randomized_hadamard(tq.randomized_hadamard_transform(dev(x), dev(s)), dev(s))
    assert np.abs(host(z) - x).max() < 1e-4


def test_polar_quantizer_object(tq):
    rng = np.random.default_rng(7)
    x = rng.standard_normal((2, 50, 128)).astype(F32)
    pq = tq.PolarQuantizer(128, bits=3, seed=42)
    idx, n = pq.quantize(dev(x))
    wi, wn = o.quantize(x, o.random_diagonal_sign(128, 42), o.gaussian_boundaries(o.gaussian_codebook(3)))
    assert idx.dtype == torch.uint8 and np.array_equal(host(idx), wi) and np.array_equal(host(n), wn)
    xh = host(pq.dequantize(idx, n))
    assert np.array_equal(xh, o.dequantize(wi, wn, o.gaussian_codebook(3), o.random_diagonal_sign(128, 42)))
    cos = (xh * x).sum(-1) / np.linalg.norm(xh, axis=-1) / np.linalg.norm(x, axis=-1)
    assert cos.mean() > 0.97


# ------------------------------------------------------------------ scores

# the default (precision=None: split operands on the matrix cores where the shape allows) and the float32
# vector kernels are held to the same bars, the reference's own
PRECS = pytest.mark.parametrize("prec", [None, "fp32"])


@PRECS
@pytest.mark.parametrize("H,S,D,bits", [(4, 64, 128, 3), (8, 256, 128, 3), (2, 16, 64, 4), (1, 128, 32, 2),
                                        (3, 1000, 128, 3), (2, 700, 128, 4), (2, 513, 128, 2), (1, 64, 128, 1)])
def test_prerot_scores_match_oracle_and_full_kernel(tq, H, S, D, bits, prec):
    rng = np.random.default_rng(8)
    c, b = tables(bits)
    s = o.random_diagonal_sign(D, 42)
    kp = o.pack_indices(rng.integers(0, 2 ** bits, size=(H, S, D)).astype(np.uint8), bits)
    kn = (rng.random((H, S)) * 10 + 1).astype(F32)
    q = rng.standard_normal((H, D)).astype(F32)
    q_rot = tq.prerotate_query(dev(q), dev(s))
    pre = host(tq.prerot_fused_qk_scores(q_rot, dev(kp), dev(kn), c, D, bits, precision=prec))
    full = host(tq.packed_fused_qk_scores(dev(q), dev(kp), dev(kn), c, dev(s), D, bits))
    want = o.prerot_fused_qk_scores(o.prerotate_query(q, s), kp, kn, c, D, bits)
    scale = max(1.0, np.abs(want).max())
    assert np.abs(pre - want).max() < 1e-5 * scale
    assert np.abs(full - want).max() < 1e-5 * scale
    assert np.abs(pre - full).max() < 1e-4 * scale                       # test_prerot.py:62-97


@PRECS
@pytest.mark.parametrize("n_kv,n_rep", [(4, 2), (2, 4), (4, 7), (1, 12), (1, 16), (1, 17)])
def test_prerot_scores_gqa(tq, n_kv, n_rep, prec):
    rng = np.random.default_rng(9)
    D, S, bits = 128, 300, 3
    c, b = tables(bits)
    kp = o.pack_indices(rng.integers(0, 8, size=(n_kv, S, D)).astype(np.uint8), bits)
    kn = (rng.random((n_kv, S)) + 0.5).astype(F32)
    qr = rng.standard_normal((n_kv * n_rep, D)).astype(F32)
    got = host(tq.prerot_fused_qk_scores(dev(qr), dev(kp), dev(kn), c, D, bits, n_rep=n_rep, precision=prec))
    want = o.prerot_fused_qk_scores(qr, kp, kn, c, D, bits, n_rep)
    assert np.abs(got - want).max() < 1e-5 * max(1.0, np.abs(want).max())
    with pytest.raises(ValueError, match="must equal n_kv_heads"):
        tq.prerot_fused_qk_scores(dev(qr[:-1]), dev(kp), dev(kn), c, D, bits, n_rep=n_rep, precision=prec)


def test_scores_on_cache_slices(tq):
    """k_packed[b, :, :total] slices of cache storage are strided views: no copy must be needed."""
    rng = np.random.default_rng(10)
    D, bits, n_kv, T_alloc, total = 128, 3, 4, 512, 300
    c, b = tables(bits)
    kp = o.pack_indices(rng.integers(0, 8, size=(2, n_kv, T_alloc, D)).astype(np.uint8), bits)
    kn = (rng.random((2, n_kv, T_alloc)) + 0.5).astype(F32)
    qr = rng.standard_normal((n_kv * 2, D)).astype(F32)
    kpt, knt = dev(kp), dev(kn)
    got = host(tq.prerot_fused_qk_scores(dev(qr), kpt[1, :, :total, :], knt[1, :, :total], c, D, bits, n_rep=2))
    want = o.prerot_fused_qk_scores(qr, kp[1, :, :total], kn[1, :, :total], c, D, bits, 2)
    assert np.abs(got - want).max() < 1e-5 * max(1.0, np.abs(want).max())


def test_dense_scores_and_softmax(tq):
    rng = np.random.default_rng(11)
    n_kv, n_rep, T, D = 4, 7, 700, 128
    K = rng.standard_normal((n_kv, T, D)).astype(np.float16)
    q = rng.standard_normal((n_kv * n_rep, D)).astype(np.float16)
    sc = 1 / math.sqrt(D)
    got = host(tq.dense_qk_scores(dev(q), dev(K), sc, n_rep=n_rep))
    want = np.einsum("grd,gtd->grt", q.reshape(n_kv, n_rep, D).astype(np.float64), K.astype(np.float64))
    want = want.reshape(n_kv * n_rep, T) * sc
    assert np.abs(got - want).max() < 1e-5 * np.abs(want).max()
    mask = np.where(rng.random((1, T)) < 0.2, -np.inf, 0.0).astype(F32)
    w = host(tq.softmax_rows(dev(got), 1.0, dev(mask)))
    ref = o._softmax64(got.astype(np.float64) + mask)
    assert np.abs(w - ref).max() < 1e-6 and np.abs(w.sum(-1) - 1).max() < 1e-5
    assert (w[:, mask[0] == -np.inf] == 0).all()


# ------------------------------------------------------------------ sparse V

def v_fixture(rng, n_kv, S, D, bits):
    c, b = tables(bits)
    s = o.random_diagonal_sign(D, 43)
    vp = o.pack_indices(rng.integers(0, 2 ** bits, size=(n_kv, S, D)).astype(np.uint8), bits)
    vn = (rng.random((n_kv, S)) + 0.1).astype(F32)
    return c, s, vp, vn


def softmax_np(x):
    e = np.exp(x - x.max(-1, keepdims=True))
    return (e / e.sum(-1, keepdims=True)).astype(F32)


@PRECS
@pytest.mark.parametrize("H,S,D,bits", [(4, 128, 128, 3), (2, 512, 128, 3), (8, 64, 64, 4), (2, 777, 256, 3),
                                        (3, 100, 32, 2), (1, 5000, 128, 3), (2, 1300, 128, 4), (2, 515, 128, 2),
                                        (1, 70, 128, 1)])
def test_sparse_v_dense_threshold(tq, H, S, D, bits, prec):
    rng = np.random.default_rng(12)
    c, s, vp, vn = v_fixture(rng, H, S, D, bits)
    w = softmax_np(rng.standard_normal((H, S)) * 3)
    want = o.sparse_v_matvec(w, vp, vn, c, s, D, bits, threshold=0.0)
    got = host(tq.sparse_v_matvec(dev(w), dev(vp), dev(vn), c, dev(s), D, bits, threshold=0.0, precision=prec))
    assert np.abs(got - want).max() / np.abs(want).max() < 1e-5         # test_sparse_v.py:47-76


@PRECS
def test_sparse_v_threshold_semantics(tq, prec):
    rng = np.random.default_rng(13)
    H, S, D, bits = 4, 2048, 128, 3
    c, s, vp, vn = v_fixture(rng, H, S, D, bits)
    w = softmax_np(rng.standard_normal((H, S)) * 5)
    args = (dev(vp), dev(vn), c, dev(s), D, bits)
    for thr in (1e-5, 1e-4, 1e-3):
        want = o.sparse_v_matvec(w, vp, vn, c, s, D, bits, threshold=thr)
        got = host(tq.sparse_v_matvec(dev(w), *args, threshold=thr, precision=prec))
        assert np.abs(got - want).max() < 1e-5 * np.abs(want).max()
    dense = host(tq.sparse_v_matvec(dev(w), *args, threshold=0.0, precision=prec))
    sp = host(tq.sparse_v_matvec(dev(w), *args, precision=prec))         # default threshold 1e-5
    assert (sp * dense).sum() / np.linalg.norm(sp) / np.linalg.norm(dense) > 0.999
    zero = host(tq.sparse_v_matvec(dev(w), *args, threshold=2.0, precision=prec))
    assert (zero == 0).all()                                             # test_sparse_v.py:150-168
    neg = host(tq.sparse_v_matvec(dev(w), *args, threshold=-1.0, precision=prec))
    assert np.array_equal(neg, dense)
    assert tq.count_active_positions(dev(w), 1e-5) == o.count_active_positions(w, 1e-5)


@PRECS
@pytest.mark.parametrize("n_kv,n_rep", [(4, 2), (2, 4), (4, 7), (2, 9), (1, 16), (1, 17)])
def test_sparse_v_gqa(tq, n_kv, n_rep, prec):
    rng = np.random.default_rng(14)
    S, D, bits = 400, 128, 3
    c, s, vp, vn = v_fixture(rng, n_kv, S, D, bits)
    w = softmax_np(rng.standard_normal((n_kv * n_rep, S)))
    want = o.sparse_v_matvec(w, vp, vn, c, s, D, bits, 0.0, n_rep)
    got = host(tq.sparse_v_matvec(dev(w), dev(vp), dev(vn), c, dev(s), D, bits, threshold=0.0, n_rep=n_rep,
                                  precision=prec))
    assert np.abs(got - want).max() < 1e-5 * np.abs(want).max()
    with pytest.raises(ValueError, match="power of 2"):
        tq.sparse_v_matvec(dev(w), dev(vp), dev(vn), c, dev(s), 96, bits)
    with pytest.raises(ValueError, match="dim > 256"):
        tq.sparse_v_matvec(dev(w), dev(vp), dev(vn), c, dev(s), 512, bits)
    with pytest.raises(ValueError, match="must equal n_kv_heads"):
        tq.sparse_v_matvec(dev(w[:-1]), dev(vp), dev(vn), c, dev(s), D, bits, n_rep=n_rep)


@pytest.mark.parametrize("S", [512, 2048, 8192, 16384])
def test_sparse_v_reference_benchmark_grid(tq, S):
    """The grid of the reference's micro-benchmark (scripts/bench_sparse_v.py:35-46, 148-171): 32 heads (MHA),
    d = 128, 3-bit values from uniform random indices, norms U(0.1, 1.1), weights = softmax(5 * N(0,1)), sequence
    lengths 512 .. 16384, thresholds 0 / 1e-5 / 1e-4.  Every point: the default sparse_v_matvec against the oracle
    to the reference's bar (tests/test_sparse_v.py:70-75), against the script's own dense composition
    (weights x packed_dequantize) by the cosine it reports, and the count of active positions."""
    rng = np.random.default_rng(S)
    H, D, bits = 32, 128, 3
    c, s, vp, vn = v_fixture(rng, H, S, D, bits)
    vn = (rng.random((H, S)) + 0.1).astype(F32)
    w = softmax_np(rng.standard_normal((H, S)) * 5)
    dw, dvp, dvn, ds = dev(w), dev(vp), dev(vn), dev(s)
    vdeq = tq.packed_dequantize(dvp.reshape(H * S, -1), dvn.reshape(-1), c, ds, D, bits).reshape(H, S, D)
    dense = host(torch.einsum("hs,hsd->hd", dw, vdeq))
    for thr in (0.0, 1e-5, 1e-4):
        want = o.sparse_v_matvec(w, vp, vn, c, s, D, bits, threshold=thr)
        got = host(tq.sparse_v_matvec(dw, dvp, dvn, c, ds, D, bits, threshold=thr))
        assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max(), (S, thr)
        cosine = float((got * dense).sum() / np.linalg.norm(got) / np.linalg.norm(dense))
        assert cosine > (0.99999 if thr == 0.0 else 0.999), (S, thr, cosine)
        assert tq.count_active_positions(dw, thr) == o.count_active_positions(w, thr)


# ------------------------------------------------------------------ flash decode

def kv_fixture(rng, n_kv, S, D, bits, outliers=False):
    c, b = tables(bits)
    ks, vs = o.random_diagonal_sign(D, 42), o.random_diagonal_sign(D, 43)
    K = rng.standard_normal((n_kv, S, D)).astype(np.float16)
    V = rng.standard_normal((n_kv, S, D)).astype(np.float16)
    if outliers:
        K[..., 7] *= 20
        V[..., 19] *= 20
    kp, kn = o.fused_quantize(K.reshape(-1, D), ks, b, D, bits)
    vp, vn = o.fused_quantize(V.reshape(-1, D), vs, b, D, bits)
    pd = o.packed_dim(D, bits)
    return (c, ks, vs, K, V, kp.reshape(n_kv, S, pd), kn.reshape(n_kv, S),
            vp.reshape(n_kv, S, pd), vn.reshape(n_kv, S))


@pytest.mark.parametrize("n_kv,n_rep,S,D,bits,bc", [(4, 1, 64, 128, 3, 16), (2, 1, 96, 128, 3, 32),
                                                    (8, 1, 256, 128, 3, 16), (2, 1, 33, 64, 4, 8),
                                                    (1, 1, 128, 32, 2, 1), (4, 2, 300, 128, 3, 16),
                                                    (2, 4, 1025, 128, 3, 16), (4, 7, 2000, 128, 3, 16)])
def test_flash_matches_oracle(tq, n_kv, n_rep, S, D, bits, bc):
    rng = np.random.default_rng(15)
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, S, D, bits)
    q = rng.standard_normal((n_kv * n_rep, D)).astype(F32)
    sc = 1 / math.sqrt(D)
    want = o.flash_attention_turboquant(o.prerotate_query(q, ks), kp, kn, vp, vn, c, c, vs, D, bits, sc, bc, n_rep)
    q_rot = tq.prerotate_query(dev(q), dev(ks))
    got = host(tq.flash_attention_turboquant(q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs),
                                             D, bits, sc, block_size=bc, n_rep=n_rep))
    assert np.abs(got - want).max() < 1e-3 * np.abs(want).max()          # test_flash_attention.py:38-137
    close(got, want)
    # equals the unfused composition on the GPU as well
    scores = tq.prerot_fused_qk_scores(q_rot, dev(kp), dev(kn), c, D, bits, n_rep=n_rep)
    w = tq.softmax_rows(scores, sc)
    comp = host(tq.sparse_v_matvec(w, dev(vp), dev(vn), c, dev(vs), D, bits, threshold=0.0, n_rep=n_rep))
    assert np.abs(got - comp).max() < 1e-3 * np.abs(comp).max()


def test_flash_argument_errors(tq):
    rng = np.random.default_rng(16)
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, 2, 32, 128, 3)
    q = dev(rng.standard_normal((2, 128)).astype(F32))
    a = (dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs))
    with pytest.raises(ValueError, match="block_size must be in 1..32"):
        tq.flash_attention_turboquant(q, *a, 128, 3, 0.1, block_size=33)
    with pytest.raises(ValueError, match="<= 128"):
        tq.flash_attention_turboquant(q, *a, 256, 3, 0.1)
    with pytest.raises(ValueError, match="must equal n_kv_heads"):
        tq.flash_attention_turboquant(q, *a, 128, 3, 0.1, n_rep=2)
    # sequences are a grid dimension: more than 65535 per call is refused before any launch
    n_seq = 65536
    offs = torch.zeros(n_seq + 1, dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError, match="at most 65535 sequences"):
        tq.flash_decode(torch.zeros((n_seq, 2, 128), device="cuda"), *a, 128, 3, 0.1, seq_offsets=offs, max_seq_len=1)


def test_flash_ragged_batch(tq):
    """A batch of sequences of different lengths in one launch (benchmark configuration 4 shape, scaled down):
    32 q heads, 8 kv heads, lengths drawn from the seed, fp16 output."""
    rng = np.random.default_rng(17)
    n_kv, n_rep, D, bits, n_seq = 8, 4, 128, 3, 5
    lens = rng.integers(40, 700, size=n_seq)
    offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, int(offs[-1]), D, bits)
    q = rng.standard_normal((n_seq, n_kv * n_rep, D)).astype(np.float16)
    sc = 1 / math.sqrt(D)
    q_rot = tq.prerotate_query(dev(q.reshape(-1, D)), dev(ks)).reshape(n_seq, n_kv * n_rep, D)
    got = tq.flash_decode(q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, sc, n_rep=n_rep,
                          seq_offsets=dev(offs), max_seq_len=int(lens.max()), out_dtype=torch.float16)
    assert got.dtype == torch.float16
    got = host(got).astype(F32)
    for i in range(n_seq):
        a, e = offs[i], offs[i + 1]
        want = o.flash_attention_turboquant(o.prerotate_query(q[i], ks), kp[:, a:e], kn[:, a:e], vp[:, a:e],
                                            vn[:, a:e], c, c, vs, D, bits, sc, 16, n_rep)
        close(got[i], want)


def test_flash_mask_and_cache_layout(tq):
    rng = np.random.default_rng(18)
    n_kv, n_rep, D, bits, B, T_alloc, total = 2, 2, 128, 3, 3, 512, 301
    sc = 1 / math.sqrt(D)
    c, b = tables(bits)
    ks, vs = o.random_diagonal_sign(D, 42), o.random_diagonal_sign(D, 43)
    kp = o.pack_indices(rng.integers(0, 8, size=(B, n_kv, T_alloc, D)).astype(np.uint8), bits)
    vp = o.pack_indices(rng.integers(0, 8, size=(B, n_kv, T_alloc, D)).astype(np.uint8), bits)
    kn = (rng.random((B, n_kv, T_alloc)) + 0.5).astype(F32)
    vn = (rng.random((B, n_kv, T_alloc)) + 0.5).astype(F32)
    q = rng.standard_normal((B, n_kv * n_rep, D)).astype(F32)
    mask = np.where(rng.random((B, 1, total)) < 0.3, -np.inf, 0.0).astype(F32)
    q_rot = tq.prerotate_query(dev(q.reshape(-1, D)), dev(ks)).reshape(B, -1, D)
    got = host(tq.flash_decode(q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, sc,
                               n_rep=n_rep, seq_len=total, mask=dev(mask)))
    for i in range(B):
        want = o.turboquant_attention_single(q[i], kp[i, :, :total], kn[i, :, :total], vp[i, :, :total],
                                             vn[i, :, :total], c, ks, c, vs, D, bits, sc, mask=mask[i])
        close(got[i], want)


# ------------------------------------------------------------------ V-only decode

@pytest.mark.parametrize("n_kv,n_rep,T,D", [(4, 7, 1000, 128), (2, 1, 64, 128), (8, 4, 513, 128), (2, 3, 300, 64),
                                           (1, 9, 257, 128)])
def test_vonly_decode_matches_oracle(tq, n_kv, n_rep, T, D):
    rng = np.random.default_rng(19)
    bits = 3
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, T, D, bits)
    q = rng.standard_normal((1, n_kv * n_rep, D)).astype(np.float16)
    sc = 1 / math.sqrt(D)
    got = host(tq.vonly_decode(dev(q), dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc, n_rep=n_rep))
    want = o.vonly_decode_attention(q[0], K, vp, vn, c, vs, D, bits, sc)
    close(got[0], want)


def test_vonly_decode_ragged_and_mask(tq):
    rng = np.random.default_rng(20)
    n_kv, n_rep, D, bits, n_seq = 4, 7, 128, 3, 4
    lens = rng.integers(10, 900, size=n_seq)
    offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, int(offs[-1]), D, bits)
    q = rng.standard_normal((n_seq, n_kv * n_rep, D)).astype(np.float16)
    sc = 1 / math.sqrt(D)
    got = host(tq.vonly_decode(dev(q), dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc, n_rep=n_rep,
                               seq_offsets=dev(offs), max_seq_len=int(lens.max())))
    for i in range(n_seq):
        a, e = offs[i], offs[i + 1]
        want = o.vonly_decode_attention(q[i], K[:, a:e], vp[:, a:e], vn[:, a:e], c, vs, D, bits, sc)
        close(got[i], want)


def test_config2_full_size(tq):
    """benchmark configuration 2 at full size: 28 q / 4 kv heads, d=128, 32768 positions; V encoded on the
    GPU (bit-exact against the oracle), then the fused V-only decode step against the oracle."""
    rng = np.random.default_rng(2)
    n_kv, n_rep, T, D, bits = 4, 7, 32768, 128, 3
    c, b = tables(bits)
    vs = o.random_diagonal_sign(D, 43)
    K = rng.standard_normal((n_kv, T, D)).astype(np.float16)
    V = rng.standard_normal((n_kv, T, D)).astype(np.float16)
    q = rng.standard_normal((1, n_kv * n_rep, D)).astype(np.float16)
    sc = 1 / math.sqrt(D)
    wp, wn = o.fused_quantize(V.reshape(-1, D), vs, b, D, bits)
    gp, gn = tq.fused_quantize(dev(V.reshape(-1, D)), dev(vs), b, D, bits)
    assert np.array_equal(host(gp), wp) and np.array_equal(host(gn), wn)
    vp, vn = gp.reshape(n_kv, T, -1), gn.reshape(n_kv, T)
    got = host(tq.vonly_decode(dev(q), dev(K), vp, vn, c, dev(vs), D, bits, sc, n_rep=n_rep))
    want = o.vonly_decode_attention(q[0], K, wp.reshape(n_kv, T, -1), wn.reshape(n_kv, T), c, vs, D, bits, sc)
    close(got[0], want)
    # unfused sparse path with the default threshold: exact against the oracle's thresholded sum.
    # On these flat weights (N(0,1) scores at 32K: most weights are near 3e-5) the threshold drops
    # about a quarter of the (head, position) pairs, so the cosine to dense is ~0.998, not the
    # 0.999 the reference quotes for peaked weights.
    scores = tq.dense_qk_scores(dev(q[0]), dev(K), 1.0, n_rep=n_rep)
    w = tq.softmax_rows(scores, sc)
    sp = host(tq.sparse_v_matvec(w, vp, vn, c, dev(vs), D, bits, threshold=1e-5, n_rep=n_rep))
    want_sp = o.vonly_decode_attention(q[0], K, wp.reshape(n_kv, T, -1), wn.reshape(n_kv, T), c, vs, D, bits,
                                       sc, threshold=1e-5)
    close(sp, want_sp)
    assert (sp * want).sum() / np.linalg.norm(sp) / np.linalg.norm(want) > 0.99


@pytest.mark.parametrize("T", [4096, 16384, 65536])
def test_config3_scores(tq, T):
    """benchmark configuration 3: pre-rotated-Q scoring over packed K, 28/4 heads, d=128."""
    rng = np.random.default_rng(3)
    n_kv, n_rep, D, bits = 4, 7, 128, 3
    c, b = tables(bits)
    ks = o.random_diagonal_sign(D, 42)
    K = rng.standard_normal((n_kv * T, D)).astype(np.float16)
    q = rng.standard_normal((n_kv * n_rep, D)).astype(np.float16)
    gp, gn = tq.fused_quantize(dev(K), dev(ks), b, D, bits)
    q_rot = tq.prerotate_query(dev(q), dev(ks))
    got = host(tq.prerot_fused_qk_scores(q_rot, gp.reshape(n_kv, T, -1), gn.reshape(n_kv, T), c, D, bits, n_rep=n_rep))
    want = o.prerot_fused_qk_scores(o.prerotate_query(q, ks), host(gp).reshape(n_kv, T, -1),
                                    host(gn).reshape(n_kv, T), c, D, bits, n_rep)
    assert got.shape == (28, T) and got.dtype == F32
    close(got, want, rel=1e-4, abs_=1e-4)


# ------------------------------------------------------------------ fp16 matrix-core variants vs float32

@pytest.mark.parametrize("n_kv,n_rep,T", [(4, 7, 2000), (8, 4, 513), (2, 16, 700), (1, 1, 64)])
def test_scores_and_sparse_v_fp16_paths(tq, n_kv, n_rep, T):
    """precision="fp16": operands rounded to half, float32 accumulation.  Scores within 2e-3 of the
    score scale, sparse-V within the attention bar; precision="fp32" stays at 1e-5."""
    rng = np.random.default_rng(21)
    D, bits = 128, 3
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, T, D, bits)
    q = rng.standard_normal((n_kv * n_rep, D)).astype(F32)
    q_rot = tq.prerotate_query(dev(q), dev(ks))
    want = o.prerot_fused_qk_scores(o.prerotate_query(q, ks), kp, kn, c, D, bits, n_rep)
    s16 = host(tq.prerot_fused_qk_scores(q_rot, dev(kp), dev(kn), c, D, bits, n_rep=n_rep, precision="fp16"))
    s32 = host(tq.prerot_fused_qk_scores(q_rot, dev(kp), dev(kn), c, D, bits, n_rep=n_rep, precision="fp32"))
    scale = np.abs(want).max()
    assert np.abs(s32 - want).max() < 1e-5 * scale
    assert np.abs(s16 - want).max() < 2e-3 * scale
    w = softmax_np(want / math.sqrt(D))
    for thr in (0.0, 1e-4):
        ws = o.sparse_v_matvec(w, vp, vn, c, vs, D, bits, thr, n_rep)
        g16 = host(tq.sparse_v_matvec(dev(w), dev(vp), dev(vn), c, dev(vs), D, bits, threshold=thr, n_rep=n_rep,
                                      precision="fp16"))
        close(g16, ws)
    z = host(tq.sparse_v_matvec(dev(w), dev(vp), dev(vn), c, dev(vs), D, bits, threshold=2.0, n_rep=n_rep,
                                precision="fp16"))
    assert (z == 0).all()
    with pytest.raises(ValueError, match="precision"):
        tq.sparse_v_matvec(dev(w), dev(vp), dev(vn), c, dev(vs), D, bits, n_rep=n_rep, precision="bf16")


@pytest.mark.parametrize("precision", ["fp16", "fp32"])
def test_flash_and_vonly_both_precisions(tq, precision):
    rng = np.random.default_rng(22)
    n_kv, n_rep, T, D, bits = 4, 7, 3000, 128, 3
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, T, D, bits, outliers=True)
    q = rng.standard_normal((n_kv * n_rep, D)).astype(np.float16)
    sc = 1 / math.sqrt(D)
    q_rot = tq.prerotate_query(dev(q), dev(ks))
    got = host(tq.flash_attention_turboquant(q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, sc,
                                             n_rep=n_rep, precision=precision))
    want = o.flash_attention_turboquant(o.prerotate_query(q, ks), kp, kn, vp, vn, c, c, vs, D, bits, sc, 16, n_rep)
    close(got, want, row_scale=True)                    # outlier channels: rows span 0.01 .. 17
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err < (1e-3 if precision == "fp16" else 1e-5), err
    got = host(tq.vonly_decode(dev(q[None]), dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc, n_rep=n_rep,
                               precision=precision))[0]
    close(got, o.vonly_decode_attention(q, K, vp, vn, c, vs, D, bits, sc), row_scale=True)


def test_config4_flash_ragged_full_heads(tq):
    """benchmark configuration 4 shape (scaled in length): 32 q / 8 kv heads, 16 sequences of ragged length,
    fp16 output, packed K and V."""
    rng = np.random.default_rng(4)
    n_kv, n_rep, D, bits, n_seq = 8, 4, 128, 3, 16
    lens = rng.integers(300, 2100, size=n_seq)
    offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, int(offs[-1]), D, bits)
    q = rng.standard_normal((n_seq, n_kv * n_rep, D)).astype(np.float16)
    sc = 1 / math.sqrt(D)
    q_rot = tq.prerotate_query(dev(q.reshape(-1, D)), dev(ks)).reshape(n_seq, n_kv * n_rep, D)
    got = host(tq.flash_decode(q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, sc, n_rep=n_rep,
                               seq_offsets=dev(offs), max_seq_len=int(lens.max()),
                               out_dtype=torch.float16)).astype(F32)
    for i in range(n_seq):
        a, e = offs[i], offs[i + 1]
        want = o.flash_attention_turboquant(o.prerotate_query(q[i], ks), kp[:, a:e], kn[:, a:e], vp[:, a:e],
                                            vn[:, a:e], c, c, vs, D, bits, sc, 16, n_rep)
        close(got[i], want)


# ------------------------------------------------------------------ chunked prefill over packed K/V

def _prefill_case(rng, n_kv, n_rep, T, n_rows, outliers=False):
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, T, 128, 3, outliers=outliers)
    q = rng.standard_normal((n_kv * n_rep, n_rows, 128)).astype(np.float16)
    if outliers:
        q[..., 7] *= 20
    return c, ks, vs, kp, kn, vp, vn, q


@pytest.mark.parametrize("n_kv,n_rep,T,n_rows,pos0", [
    (2, 2, 300, 300, 0),        # whole prompt in one chunk, ragged everywhere
    (2, 4, 1000, 256, 744),     # tail chunk of exactly one workgroup of rows
    (1, 1, 777, 130, 500),      # chunk in the middle of a longer cache (positions past it are ignored)
    (2, 2, 2500, 513, 1987),    # three row blocks, several splits
])
def test_prefill_attention_matches_oracle(tq, n_kv, n_rep, T, n_rows, pos0):
    rng = np.random.default_rng(51)
    c, ks, vs, kp, kn, vp, vn, q = _prefill_case(rng, n_kv, n_rep, T, n_rows)
    sc = 1 / math.sqrt(128)
    want = o.prefill_attention(q, kp, kn, vp, vn, c, c, ks, vs, 128, 3, sc, pos0, n_rep)
    got = tq.prefill_attention(dev(q), dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(ks), dev(vs), 128, 3, sc,
                               n_rep=n_rep, q_pos0=pos0, out_dtype=torch.float32)
    assert got.shape == (n_kv * n_rep, n_rows, 128)
    close(host(got).reshape(-1, 128), want.reshape(-1, 128))      # N(0,1) data, no outlier channels: elementwise 2e-3 / 1e-3
    rel = np.abs(host(got) - want).max() / np.abs(want).max()
    assert rel < 1e-3, rel


def test_prefill_attention_noncausal_fp16_out_and_outliers(tq):
    """1 % outlier channels (x20) in K, V and q as in benchmark configuration 5; fp16 output; and the
    non-causal form, where every row sees every position."""
    rng = np.random.default_rng(52)
    n_kv, n_rep, T, n_rows = 2, 4, 1500, 200
    c, ks, vs, kp, kn, vp, vn, q = _prefill_case(rng, n_kv, n_rep, T, n_rows, outliers=True)
    sc = 1 / math.sqrt(128)
    for causal in (True, False):
        want = o.prefill_attention(q, kp, kn, vp, vn, c, c, ks, vs, 128, 3, sc, T - n_rows, n_rep, causal=causal)
        got = tq.prefill_attention(dev(q), dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(ks), dev(vs), 128, 3, sc,
                                   n_rep=n_rep, causal=causal)
        assert got.dtype == torch.float16
        err = np.abs(host(got).astype(np.float64) - want)
        scale = np.abs(want).max(axis=-1, keepdims=True)
        assert (err <= 1e-3 + 2.5e-3 * scale).all(), (err / scale).max()   # 2e-3 + fp16 rounding of the output (4.9e-4)


def test_prefill_attention_fp16_query_flag(tq):
    """fp16_query=True (the rotated query as one fp16 number per element, a third fewer matrix instructions) meets
    the elementwise bar on N(0,1) data -- and does NOT meet the outlier test's bar on data with x20 outlier channels,
    which is why it is off by default: the default path must keep passing that test with its remainder in."""
    rng = np.random.default_rng(51)
    n_kv, n_rep, T, n_rows, pos0 = 2, 4, 1000, 256, 744
    c, ks, vs, kp, kn, vp, vn, q = _prefill_case(rng, n_kv, n_rep, T, n_rows)
    sc = 1 / math.sqrt(128)
    want = o.prefill_attention(q, kp, kn, vp, vn, c, c, ks, vs, 128, 3, sc, pos0, n_rep)
    got = tq.prefill_attention(dev(q), dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(ks), dev(vs), 128, 3, sc,
                               n_rep=n_rep, q_pos0=pos0, out_dtype=torch.float32, fp16_query=True)
    close(host(got).reshape(-1, 128), want.reshape(-1, 128))
    rng = np.random.default_rng(52)
    n_kv, n_rep, T, n_rows = 2, 4, 1500, 200
    c, ks, vs, kp, kn, vp, vn, q = _prefill_case(rng, n_kv, n_rep, T, n_rows, outliers=True)
    want = o.prefill_attention(q, kp, kn, vp, vn, c, c, ks, vs, 128, 3, sc, T - n_rows, n_rep)
    errs = {}
    for flag in (False, True):
        got = tq.prefill_attention(dev(q), dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(ks), dev(vs), 128, 3, sc,
                                   n_rep=n_rep, out_dtype=torch.float32, fp16_query=flag)
        err = np.abs(host(got).astype(np.float64) - want)
        scale = np.abs(want).max(axis=-1, keepdims=True)
        errs[flag] = float(((err - 1e-3) / scale).max())
    assert errs[False] <= 2e-3, errs
    assert errs[True] > 2e-3, errs                    # the flag is refused by the bar of the outlier test


def test_prefill_attention_equals_decode_rows(tq):
    """Each row of a prefill chunk is one decode step over its prefix: compare with the
    float32 flash decode kernel of this library (independent code path)."""
    rng = np.random.default_rng(53)
    n_kv, n_rep, T, n_rows = 2, 2, 640, 64
    c, ks, vs, kp, kn, vp, vn, q = _prefill_case(rng, n_kv, n_rep, T, n_rows)
    sc = 1 / math.sqrt(128)
    got = host(tq.prefill_attention(dev(q), dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(ks), dev(vs), 128, 3, sc,
                                    n_rep=n_rep, out_dtype=torch.float32))
    for i in (0, 17, 63):
        L = T - n_rows + i + 1
        q_rot = tq.prerotate_query(dev(q[:, i]), dev(ks))
        ref = host(tq.flash_attention_turboquant(q_rot, dev(kp[:, :L]), dev(kn[:, :L]), dev(vp[:, :L]), dev(vn[:, :L]),
                                                 c, c, dev(vs), 128, 3, sc, n_rep=n_rep, precision="fp32"))
        close(got[:, i], ref, row_scale=True)


def test_prefill_attention_argument_errors(tq):
    rng = np.random.default_rng(54)
    c, ks, vs, kp, kn, vp, vn, q = _prefill_case(rng, 2, 2, 128, 16)
    args = (dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(ks), dev(vs))
    with pytest.raises(ValueError):
        tq.prefill_attention(dev(q), *args, 128, 3, 0.1, n_rep=3)                 # 4 q heads != 2 * 3
    with pytest.raises(ValueError):
        tq.prefill_attention(dev(q), *args, 128, 3, 0.1, n_rep=2, q_pos0=500)     # chunk starts past the cache
    with pytest.raises(RuntimeError):
        tq.prefill_attention(dev(q[..., :64]), dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(ks[:64]), dev(vs[:64]),
                             64, 3, 0.1, n_rep=2)                                 # no kernel for d = 64
    empty = tq.prefill_attention(dev(q[:, :0]), *args, 128, 3, 0.1, n_rep=2, q_pos0=0)
    assert empty.shape == (4, 0, 128)


# ------------------------------------------------------------------ HIP graph capture

def test_decode_ops_replay_under_hip_graph(tq):
    """The ops only launch kernels on torch's current stream (no allocation once the workspace exists,
    no memset nodes), so a decode step can be captured once and replayed.  Every replay - with the
    inputs rewritten in place and eager work in between - must reproduce the eager result."""
    rng = np.random.default_rng(90)
    n_kv, n_rep, T, D, bits = 4, 7, 2048, 128, 3
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, T, D, bits)
    sc = 1 / math.sqrt(D)
    q = dev(rng.standard_normal((1, n_kv * n_rep, D)).astype(np.float16))
    Kd, vpd, vnd, kpd, knd = dev(K), dev(vp), dev(vn), dev(kp), dev(kn)
    vsd, ksd = dev(vs), dev(ks)

    def step():
        a = tq.vonly_decode(q, Kd, vpd, vnd, c, vsd, D, bits, sc, n_rep=n_rep)
        q_rot = tq.prerotate_query(q[0], ksd)
        b = tq.flash_attention_turboquant(q_rot, kpd, knd, vpd, vnd, c, c, vsd, D, bits, sc, n_rep=n_rep)
        return a, b

    step()                                                    # warm-up: workspace, tables
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        step()
        with torch.cuda.graph(graph, stream=side):
            ga, gb = step()
    torch.cuda.current_stream().wait_stream(side)
    for it in range(4):
        q.copy_(dev(rng.standard_normal((1, n_kv * n_rep, D)).astype(np.float16)))
        if it == 2:
            Kd.mul_(0.5)                                       # the graph reads the buffers, not a snapshot
        graph.replay()
        torch.cuda.synchronize()
        ra, rb = ga.clone(), gb.clone()
        ea, eb = step()                                        # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(ra, ea) and torch.equal(rb, eb), it


# ------------------------------------------------------------------ streaming V-only kernel (several blocks per workgroup)

@pytest.mark.parametrize("n_seq,n_kv,n_rep,T,blocks", [(8, 8, 2, 4096, 2), (8, 8, 2, 6144, 3), (4, 8, 4, 16384, 4)])
def test_vonly_decode_streaming_blocks(tq, n_seq, n_kv, n_rep, T, blocks):
    """Unmasked caches with more than 256 tiles of 512 positions take the streaming kernel, in which a
    workgroup runs through `blocks` consecutive tiles with an online softmax.  Value norms jump by
    factors of 2^+-6 between tiles and the largest scores sit in different tiles per head, so both the
    running-maximum rescale and the change of the power-of-two norm scale are exercised."""
    assert (T // 512) * n_kv * n_seq // 256 == blocks
    rng = np.random.default_rng(95)
    D, bits = 128, 3
    c, b = tables(bits)
    vs = o.random_diagonal_sign(D, 43)
    sc = 1 / math.sqrt(D)
    K = rng.standard_normal((n_seq, n_kv, T, D)).astype(np.float16)
    V = rng.standard_normal((n_seq, n_kv, T, D)).astype(np.float32)
    V *= (2.0 ** rng.integers(-6, 7, size=(n_seq, n_kv, T // 512, 1, 1))).repeat(512, axis=2).reshape(n_seq, n_kv, T, 1, 1)[..., 0]
    q = rng.standard_normal((n_seq, n_kv * n_rep, D)).astype(np.float16)
    Kd, qd = dev(K), dev(q)
    vp, vn = tq.fused_quantize(dev(V.astype(np.float16)).reshape(-1, D), dev(vs), b, D, bits)
    vp, vn = vp.reshape(n_seq, n_kv, T, -1), vn.reshape(n_seq, n_kv, T)
    got = host(tq.vonly_decode(qd, Kd, vp, vn, c, dev(vs), D, bits, sc, n_rep=n_rep))
    ref32 = host(tq.vonly_decode(qd, Kd, vp, vn, c, dev(vs), D, bits, sc, n_rep=n_rep, precision="fp32"))
    hp, hn = host(vp), host(vn)
    for sidx in range(0, n_seq, max(1, n_seq // 2)):             # oracle on a subset of the sequences
        want = o.vonly_decode_attention(q[sidx], K[sidx], hp[sidx], hn[sidx], c, vs, D, bits, sc)
        close(got[sidx], want, row_scale=True)
    close(got.reshape(-1, D), ref32.reshape(-1, D), row_scale=True)   # every sequence against the float32 kernels


# ------------------------------------------------------------------ seeded sweep over decode shapes

def _draw_decode_case(seed):
    """One decode-attention case drawn from the seed: head counts (including group sizes that do not
    divide the 16-row matrix tile evenly), a ragged batch or a cache-layout batch, lengths from 1
    to a few thousand (log-uniform, so tile boundaries, single positions and multi-tile sequences
    all occur), an optional additive mask per sequence or per head, and the query dtype."""
    rng = np.random.default_rng(1000 + seed)
    n_kv = int(rng.choice([1, 2, 3, 4, 5, 8]))
    n_rep = int(rng.choice([1, 2, 3, 4, 5, 7, 8, 12, 16]))
    ragged = bool(rng.integers(0, 2))
    n_seq = int(rng.integers(1, 5))
    hi = 3000 if n_kv * n_rep <= 32 else 1200
    lens = np.exp(rng.uniform(0.0, math.log(hi), size=n_seq)).astype(np.int64).clip(1, hi)
    if not ragged:
        lens[:] = lens[0]
    mask_kind = ["none", "seq", "head"][int(rng.integers(0, 3))] if not ragged else "none"
    qdt = [np.float16, np.float32][int(rng.integers(0, 2))]
    return rng, n_kv, n_rep, ragged, n_seq, lens, mask_kind, qdt


def _draw_mask(rng, kind, n_seq, n_q, T):
    if kind == "none":
        return None
    shape = (n_seq, 1, T) if kind == "seq" else (n_seq, n_q, T)
    m = np.where(rng.random(shape) < 0.3, -np.inf, 0.0).astype(F32)
    m[..., int(rng.integers(0, T))] = 0.0          # no row fully masked
    return m + (rng.standard_normal(shape) * 0.5).astype(F32) * np.isfinite(m)


@pytest.mark.parametrize("seed", range(24))
def test_decode_sweep_vonly_and_flash(tq, seed):
    """vonly_decode and flash_decode (both precisions) on shapes drawn from the seed, each sequence
    checked against the oracle's single-sequence functions."""
    rng, n_kv, n_rep, ragged, n_seq, lens, mask_kind, qdt = _draw_decode_case(seed)
    D, bits, sc = 128, 3, 1 / math.sqrt(128)
    n_q = n_kv * n_rep
    print(f"seed {seed}: n_kv {n_kv} n_rep {n_rep} ragged {ragged} lens {lens.tolist()} mask {mask_kind} "
          f"q {np.dtype(qdt).name}", flush=True)
    q = rng.standard_normal((n_seq, n_q, D)).astype(qdt)
    if ragged:
        offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, int(offs[-1]), D, bits)
        kw = dict(seq_offsets=dev(offs), max_seq_len=int(lens.max()))
        per_seq = [tuple(a[:, offs[i]:offs[i + 1]] for a in (K, kp, kn, vp, vn)) for i in range(n_seq)]
        dK, dkp, dkn, dvp, dvn = (dev(a) for a in (K, kp, kn, vp, vn))
        mask = None
    else:
        T = int(lens[0])
        T_alloc = T + int(rng.integers(0, 70))
        c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_seq * n_kv, T_alloc, D, bits)
        K, kp, kn, vp, vn = (a.reshape(n_seq, n_kv, *a.shape[1:]) for a in (K, kp, kn, vp, vn))
        kw = dict(seq_len=T)
        per_seq = [tuple(a[i, :, :T] for a in (K, kp, kn, vp, vn)) for i in range(n_seq)]
        dK, dkp, dkn, dvp, dvn = (dev(a) for a in (K, kp, kn, vp, vn))
        mask = _draw_mask(rng, mask_kind, n_seq, n_q, T)
        if mask is not None:
            kw["mask"] = dev(mask)
    q_rot = tq.prerotate_query(dev(q.reshape(-1, D)), dev(ks)).reshape(n_seq, n_q, D)
    for precision in ("fp16", "fp32"):
        gv = host(tq.vonly_decode(dev(q), dK, dvp, dvn, c, dev(vs), D, bits, sc, n_rep=n_rep,
                                  precision=precision, **kw))
        gf = host(tq.flash_decode(q_rot, dkp, dkn, dvp, dvn, c, c, dev(vs), D, bits, sc, n_rep=n_rep,
                                  precision=precision, **kw))
        for i in range(n_seq):
            Ki, kpi, kni, vpi, vni = per_seq[i]
            mi = None if mask is None else np.broadcast_to(mask[i], (n_q, mask.shape[-1]))
            close(gv[i], o.vonly_decode_attention(q[i], Ki, vpi, vni, c, vs, D, bits, sc, mask=mi))
            close(gf[i], o.turboquant_attention_single(q[i].astype(F32), kpi, kni, vpi, vni, c, ks, c, vs,
                                                       D, bits, sc, mask=mi))


@pytest.mark.parametrize("seed", range(12))
def test_decode_sweep_scores_and_sparse_v(tq, seed):
    """The two unfused kernels on drawn shapes: scores of packed K (float32 kernel held to float32
    rounding, matrix-core kernel to 1e-3 of the row scale) and the thresholded V sum."""
    rng, n_kv, n_rep, _, _, lens, _, _ = _draw_decode_case(100 + seed)
    D, bits, T = 128, 3, int(lens[0])
    n_q = n_kv * n_rep
    print(f"seed {seed}: n_kv {n_kv} n_rep {n_rep} T {T}", flush=True)
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, T, D, bits)
    q_rot = o.prerotate_query(rng.standard_normal((n_q, D)).astype(F32), ks)
    want = o.prerot_fused_qk_scores(q_rot, kp, kn, c, D, bits, n_rep)
    got32 = host(tq.prerot_fused_qk_scores(dev(q_rot), dev(kp), dev(kn), c, D, bits, n_rep))
    # float32 sums of 128 terms: the rounding error goes with the size of the terms, i.e. with the scale of the
    # scores, also where a score itself is small through cancellation
    close(got32, want, rel=1e-5, abs_=max(1e-5, 1e-6 * float(np.abs(want).max())))
    got16 = host(tq.prerot_fused_qk_scores(dev(q_rot), dev(kp), dev(kn), c, D, bits, n_rep, precision="fp16"))
    close(got16, want, rel=1e-3, abs_=1e-3 * float(np.abs(want).max()))
    w = rng.random((n_q, T)) ** 8                      # float64: a single tiny weight must not underflow to 0 / 0
    w = (w / w.sum(axis=-1, keepdims=True)).astype(F32)
    thr = float(rng.choice([0.0, 1e-5, 1e-3]))
    wantv = o.sparse_v_matvec(w, vp, vn, c, vs, D, bits, threshold=thr, n_rep=n_rep)
    for precision in ("fp32", "fp16", None):
        gotv = host(tq.sparse_v_matvec(dev(w), dev(vp), dev(vn), c, dev(vs), D, bits, threshold=thr,
                                       n_rep=n_rep, precision=precision))
        close(gotv, wantv)
        if precision != "fp16":                         # the reference's bar (tests/test_sparse_v.py:70-75)
            assert np.abs(gotv - wantv).max() <= 1e-5 * np.abs(wantv).max()
    s32 = host(tq.prerot_fused_qk_scores(dev(q_rot), dev(kp), dev(kn), c, D, bits, n_rep, precision="fp32"))
    close(s32, want, rel=1e-5, abs_=max(1e-5, 1e-6 * float(np.abs(want).max())))


@pytest.mark.parametrize("seed", range(10))
def test_prefill_sweep(tq, seed):
    """Prefill attention on drawn shapes: chunk length, chunk position inside the cache (tail, middle,
    start), cache allocation longer than the attended length, group size, causal or not."""
    rng = np.random.default_rng(2000 + seed)
    n_kv = int(rng.choice([1, 2, 3]))
    n_rep = int(rng.choice([1, 2, 4, 7]))
    kv_len = int(np.exp(rng.uniform(math.log(2), math.log(2600))))
    n_rows = int(rng.integers(1, min(kv_len, 600) + 1))
    causal = bool(rng.integers(0, 4))
    where = int(rng.integers(0, 3))
    pos0 = [kv_len - n_rows, int(rng.integers(0, kv_len - n_rows + 1)), 0][where]
    T_alloc = kv_len + int(rng.integers(0, 100))
    print(f"seed {seed}: n_kv {n_kv} n_rep {n_rep} kv_len {kv_len} alloc {T_alloc} rows {n_rows} pos0 {pos0} "
          f"causal {causal}", flush=True)
    c, ks, vs, kp, kn, vp, vn, q = _prefill_case(rng, n_kv, n_rep, T_alloc, n_rows)
    sc = 1 / math.sqrt(128)
    want = o.prefill_attention(q, kp[:, :kv_len], kn[:, :kv_len], vp[:, :kv_len], vn[:, :kv_len], c, c, ks, vs,
                               128, 3, sc, pos0, n_rep, causal=causal)
    got = tq.prefill_attention(dev(q), dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(ks), dev(vs), 128, 3, sc,
                               n_rep=n_rep, kv_len=kv_len, q_pos0=pos0, causal=causal, out_dtype=torch.float32)
    close(host(got).reshape(-1, 128), want.reshape(-1, 128), row_scale=True)


@pytest.mark.parametrize("seed", range(8))
def test_encode_sweep(tq, seed):
    """encode_into / dequant_into on drawn group layouts (row counts that do and do not meet the
    streaming kernel's 16-row granularity, strides, offsets) and input scales: bit-exact."""
    rng = np.random.default_rng(3000 + seed)
    c, b = tables(3)
    s = o.random_diagonal_sign(128, 42 + seed)
    G = int(rng.integers(1, 6))
    R = int(rng.choice([1, 5, 16, 17, 48, 64, 250, 1024]))
    off = int(rng.integers(0, 40))
    alloc = off + R + int(rng.integers(0, 40))
    dt = [np.float16, np.float32][int(rng.integers(0, 2))]
    variant = ["mlx", "metal"][int(rng.integers(0, 2))]
    print(f"seed {seed}: G {G} R {R} off {off} alloc {alloc} {np.dtype(dt).name} {variant}", flush=True)
    x = (rng.standard_normal((G, R, 128)) * np.exp(rng.uniform(-6, 6, size=(G, R, 1)))).astype(dt)
    packed = torch.zeros((G, alloc, 13), dtype=torch.int32, device="cuda").view(torch.uint32)
    norms = torch.zeros((G, alloc), dtype=torch.float32, device="cuda")
    tq.encode_into(dev(x), dev(s), b, packed, norms, n_groups=G, rows_per_group=R, packed_group_stride=alloc,
                   norms_group_stride=alloc, dim=128, bits=3, packed_row_offset=off, norms_row_offset=off,
                   variant=variant)
    wp, wn = o.fused_quantize(x.reshape(-1, 128), s, b, 128, 3, variant)
    hp, hn = host(packed), host(norms)
    assert np.array_equal(hp[:, off:off + R], wp.reshape(G, R, 13))
    assert np.array_equal(hn[:, off:off + R], wn.reshape(G, R))
    assert (hp[:, :off] == 0).all() and (hp[:, off + R:] == 0).all()
    out = torch.zeros((G, alloc, 128), dtype=torch.float16, device="cuda")
    tq.dequant_into(packed, norms, c, dev(s), out, n_groups=G, rows_per_group=R, packed_group_stride=alloc,
                    norms_group_stride=alloc, out_group_stride=alloc, dim=128, bits=3, packed_row_offset=off,
                    norms_row_offset=off, out_row_offset=off)
    want = torch.from_numpy(o.packed_dequantize(wp, wn, c, s, 128, 3)).to(torch.float16).reshape(G, R, 128)
    assert torch.equal(out[:, off:off + R].cpu(), want)


# ------------------------------------------------------------------ streaming flash pass

def _flash_plan(tq, n_seq, n_kv, max_len, ragged, masked=False):
    from tqhip import _lib
    return _lib.load().tq_flash_decode_plan(n_seq, n_kv, max_len, int(ragged), int(masked))


def test_flash_streaming_pass_ragged(tq):
    """A ragged batch large enough for the streaming pass (several 256-position steps per workgroup):
    sequences start at arbitrary rows (every misalignment of the 52-byte rows against 16 bytes),
    lengths end inside a step, inside a wave's 64 rows and one row past a step."""
    rng = np.random.default_rng(61)
    n_kv, n_rep, D, bits = 8, 4, 128, 3
    lens = np.array([4097, 2561, 1025, 7000, 1, 3333, 5121, 6143])
    n_seq = len(lens)
    assert _flash_plan(tq, n_seq, n_kv, int(lens.max()), True) >= 2
    offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    assert len({int(o) % 4 for o in offs[:-1]}) == 4          # all four row misalignments occur
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, int(offs[-1]), D, bits)
    q = rng.standard_normal((n_seq, n_kv * n_rep, D)).astype(F32)
    sc = 1 / math.sqrt(D)
    q_rot = tq.prerotate_query(dev(q.reshape(-1, D)), dev(ks)).reshape(n_seq, n_kv * n_rep, D)
    got = host(tq.flash_decode(q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, sc, n_rep=n_rep,
                               seq_offsets=dev(offs), max_seq_len=int(lens.max())))
    for i in range(n_seq):
        a, e = offs[i], offs[i + 1]
        want = o.flash_attention_turboquant(o.prerotate_query(q[i], ks), kp[:, a:e], kn[:, a:e], vp[:, a:e],
                                            vn[:, a:e], c, c, vs, D, bits, sc, 16, n_rep)
        close(got[i], want)


@pytest.mark.parametrize("n_seq,n_kv,n_rep,T,outliers", [(2, 8, 2, 16500, False), (1, 4, 7, 70000, False),
                                                          (3, 8, 1, 12289, True), (1, 8, 4, 24001, False)])
def test_flash_streaming_pass_cache_layout(tq, n_seq, n_kv, n_rep, T, outliers):
    """Cache layout [n_seq, n_kv, T_alloc, *] with a valid length that is not a multiple of anything;
    value norms spread over six decades so that the running power-of-two scale moves between steps."""
    rng = np.random.default_rng(62)
    D, bits, T_alloc = 128, 3, T + 37
    assert _flash_plan(tq, n_seq, n_kv, T, False) >= 2
    c, b = tables(bits)
    ks, vs = o.random_diagonal_sign(D, 42), o.random_diagonal_sign(D, 43)
    kp = o.pack_indices(rng.integers(0, 8, size=(n_seq, n_kv, T_alloc, D)).astype(np.uint8), bits)
    vp = o.pack_indices(rng.integers(0, 8, size=(n_seq, n_kv, T_alloc, D)).astype(np.uint8), bits)
    kn = (rng.random((n_seq, n_kv, T_alloc)) * 12 + 6).astype(F32)
    vn = (rng.random((n_seq, n_kv, T_alloc)) + 0.5).astype(F32)
    if outliers:
        vn *= np.exp(rng.uniform(-7, 7, size=vn.shape)).astype(F32)
    q = rng.standard_normal((n_seq, n_kv * n_rep, D)).astype(F32)
    sc = 1 / math.sqrt(D)
    q_rot = tq.prerotate_query(dev(q.reshape(-1, D)), dev(ks)).reshape(n_seq, -1, D)
    got = host(tq.flash_decode(q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, sc,
                               n_rep=n_rep, seq_len=T))
    for i in range(n_seq):
        want = o.turboquant_attention_single(q[i], kp[i, :, :T], kn[i, :, :T], vp[i, :, :T], vn[i, :, :T],
                                             c, ks, c, vs, D, bits, sc)
        close(got[i], want, row_scale=outliers)


def test_flash_plan_masked_and_small_batches_take_the_tile_pass(tq):
    assert _flash_plan(tq, 1, 4, 4096, False) == 0
    assert _flash_plan(tq, 16, 8, 32768, True, masked=True) == 0
    assert _flash_plan(tq, 16, 8, 32768, True) == 4
    assert _flash_plan(tq, 1, 8, 131072, False) == 8
    # one four-wave workgroup per CU where three steps reach that and two would leave 384 workgroups
    assert _flash_plan(tq, 1, 8, 24576, False) == 3
    assert _flash_plan(tq, 1, 8, 20480, False) == 3
    assert _flash_plan(tq, 1, 8, 32768, False) == 2
    assert _flash_plan(tq, 1, 8, 36864, False) == 3
    assert _flash_plan(tq, 1, 8, 18432, False) == 3
    assert _flash_plan(tq, 1, 8, 16384, False) == 0
    # more than 512 workgroups at any step count: whole rounds (1024 workgroups of five steps, not 640 of eight)
    assert _flash_plan(tq, 16, 8, 10240, False) == 5


def test_encode_fp16_denormal_and_tiny_inputs(tq):
    """fp16 inputs whose elements are mostly subnormal halves (scale 1e-5) or exactly representable tiny
    values: the streaming encoder widens them inside mixed-precision multiplies and must still be
    bit-exact, norms included."""
    rng = np.random.default_rng(71)
    c, b = tables(3)
    s = o.random_diagonal_sign(128, 43)
    x = (rng.standard_normal((640, 128)) * np.repeat([1e-5, 3e-5, 1e-4, 6e-8], 160)[:, None]).astype(np.float16)
    x[5] = 0
    x[6, 3] = np.float16(6e-8)          # one subnormal element, everything else zero
    x[6, :3] = 0; x[6, 4:] = 0
    assert (np.abs(x[x != 0]).astype(np.float32) < 6.1e-5).mean() > 0.5
    wp, wn = o.fused_quantize(x, s, b, 128, 3)
    gp, gn = tq.fused_quantize(dev(x), dev(s), b, 128, 3)
    assert np.array_equal(host(gp), wp) and np.array_equal(host(gn), wn)


# ------------------------------------------------------------------ committed closed-form vectors

def _golden_cases():
    import json
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "kat_vectors.json")
    with open(path) as f:
        return json.load(f)["cases"]


@pytest.mark.parametrize("case", _golden_cases(), ids=lambda c: c["name"])
def test_kernels_reproduce_closed_form_vectors(tq, case):
    """The committed known answers (exact rational arithmetic on the Hadamard closed form) through the
    C ABI: encode bit-exact in both threshold variants and from fp16 and fp32 inputs, alone (generic
    kernel) and as 48 repeated rows (streaming kernel for d = 128 / 3-bit); dequant to float32 rounding."""
    d, bits = case["dim"], case["bits"]
    x = np.array(case["x"], np.float32)
    s = np.array(case["signs"], np.float32)
    c, b = tables(bits)
    want_words = np.array([int(w, 16) for w in case["packed_hex"]], np.uint32)
    for variant in ("mlx", "metal"):
        for dt in (np.float32, np.float16):
            for reps in (1, 48):
                xs = np.repeat(x[None, :], reps, axis=0).astype(dt)
                gp, gn = tq.fused_quantize(dev(xs), dev(s), b, d, bits, variant=variant)
                gp, gn = host(gp), host(gn)
                assert (gp == want_words[None, :]).all(), (variant, dt, reps)
                assert (gn == np.float32(case["norm"])).all()
    p = dev(np.repeat(want_words[None, :], 48, axis=0))
    n = dev(np.full(48, case["norm"], np.float32))
    want = np.array(case["dequant"])
    tol = 2e-6 * max(1.0, np.abs(want).max())
    for reps in (1, 48):
        deq = host(tq.packed_dequantize(p[:reps], n[:reps], c, dev(s), d, bits)).astype(np.float64)
        assert np.abs(deq - want[None, :]).max() <= tol


@pytest.mark.parametrize("n_kv,n_rep", [(8, 1), (4, 5), (2, 16)])
def test_flash_streaming_pass_group_sizes_and_leading_offset(tq, n_kv, n_rep):
    """Streaming pass with 1, 5 and 16 query heads per kv head, and a batch whose first sequence does not
    start at row 0 (every block misaligned against 16 bytes by the same amount)."""
    rng = np.random.default_rng(63 + n_rep)
    D, bits = 128, 3
    n_seq = 64 // n_kv                                 # 64 (sequence, kv head) pairs x 17 steps of 256 positions
    lens = rng.integers(4000, 4600, size=n_seq)
    offs = (3 + np.concatenate([[0], np.cumsum(lens)])).astype(np.int32)
    assert _flash_plan(tq, n_seq, n_kv, int(lens.max()), True) >= 2
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, int(offs[-1]), D, bits)
    q = rng.standard_normal((n_seq, n_kv * n_rep, D)).astype(F32)
    sc = 1 / math.sqrt(D)
    q_rot = tq.prerotate_query(dev(q.reshape(-1, D)), dev(ks)).reshape(n_seq, n_kv * n_rep, D)
    got = host(tq.flash_decode(q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, sc, n_rep=n_rep,
                               seq_offsets=dev(offs), max_seq_len=int(lens.max())))
    for i in range(0, n_seq, max(1, n_seq // 6)):
        a, e = offs[i], offs[i + 1]
        want = o.flash_attention_turboquant(o.prerotate_query(q[i], ks), kp[:, a:e], kn[:, a:e], vp[:, a:e],
                                            vn[:, a:e], c, c, vs, D, bits, sc, 16, n_rep)
        close(got[i], want)


@pytest.mark.parametrize("n_seq,n_kv,n_rep,T,masked", [
    (1, 8, 4, 5003, False),      # 80 eight-wave tiles: workgroups of four waves over 256-position tiles
    (1, 8, 4, 10007, False),     # 160: one eight-wave workgroup per CU
    (2, 8, 2, 9001, True),       # 288, masked: two eight-wave workgroups per CU
    (1, 2, 16, 257, False), (3, 1, 7, 256, True)])
def test_flash_tile_pass_workgroup_shapes(tq, n_seq, n_kv, n_rep, T, masked):
    """The three shapes of the packed tile pass in its flash mode (chosen by how many tiles the call has), each
    against the oracle, lengths that end inside a wave's rows and one row into a tile, with and without a mask."""
    rng = np.random.default_rng(5 * T + n_rep)
    D, bits, sc = 128, 3, 1 / math.sqrt(128)
    n_q = n_kv * n_rep
    assert _flash_plan(tq, n_seq, n_kv, T, False, masked) == 0       # the tile pass, not the streaming one
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_seq * n_kv, T + 9, D, bits)
    kp, kn, vp, vn = (a.reshape(n_seq, n_kv, *a.shape[1:]) for a in (kp, kn, vp, vn))
    q = rng.standard_normal((n_seq, n_q, D)).astype(F32)
    mask = _draw_mask(rng, "head" if masked else "none", n_seq, n_q, T)
    kw = {} if mask is None else dict(mask=dev(mask))
    q_rot = tq.prerotate_query(dev(q.reshape(-1, D)), dev(ks)).reshape(n_seq, n_q, D)
    got = host(tq.flash_decode(q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, sc, n_rep=n_rep,
                               seq_len=T, **kw))
    for i in range(n_seq):
        mi = None if mask is None else np.broadcast_to(mask[i], (n_q, T))
        want = o.turboquant_attention_single(q[i], kp[i, :, :T], kn[i, :, :T], vp[i, :, :T], vn[i, :, :T], c, ks, c, vs,
                                             D, bits, sc, mask=mi)
        close(got[i], want)


def encoded_kv_on_gpu(tq, g, n_kv, n_rows, bits, signs, outlier_channel=None):
    """K or V of a benchmark configuration at full size: seeded N(0,1) fp16 rows drawn on the GPU (optionally one
    channel scaled x20), encoded by the library's own encoder -- whose words and norms at this size are compared
    with the oracle bit for bit in test_config5_full_size_encode_paths_agree.  Returns (packed (n_kv, n_rows, pdim)
    uint32, norms (n_kv, n_rows) float32) on the GPU."""
    c, b = tables(bits)
    packed, norms = [], []
    for h in range(n_kv):
        x = torch.randn((n_rows, 128), generator=g, device="cuda", dtype=torch.float32).to(torch.float16)
        if outlier_channel is not None:
            x[:, outlier_channel] *= 20
        p, n = tq.fused_quantize(x, signs, b, 128, bits)
        packed.append(p)
        norms.append(n)
        del x
    return torch.stack(packed), torch.stack(norms)


def test_config4_full_size_paths_agree(tq):
    """benchmark configuration 4 at full size (16 sequences of 4096..32768 positions, 32 q / 8 kv heads, fp16
    out): the streaming pass, the one-tile-per-workgroup pass (forced by an all-zero mask) and the float32
    kernels are three separate code paths and must agree; the two shortest sequences and the LONGEST one (the most
    steps of the streaming pass) are also checked against the oracle.  Data as the configuration states it: K and V
    are the encoder's output for seeded N(0,1) fp16 rows.  Tolerances: 2e-3 of the row maximum (the reference's own
    measure, tests/test_flash_attention.py) for fp16-operand against float32 arithmetic, 2.5e-3 where the fp16
    rounding of the OUTPUT (at most 4.9e-4 of an element) comes on top; the absolute term is 1e-4 here, not 1e-3:
    the rows of a flat softmax over thousands of N(0,1) values are of size 0.01 - 0.05, where 1e-3 would pass
    anything."""
    rng = np.random.default_rng(4)
    n_kv, n_rep, D, bits, n_seq = 8, 4, 128, 3, 16
    lens = rng.integers(4096, 32769, size=n_seq)
    offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    total, max_len = int(offs[-1]), int(lens.max())
    assert _flash_plan(tq, n_seq, n_kv, max_len, True) >= 2
    c, b = tables(bits)
    ks, vs = o.random_diagonal_sign(D, 42), o.random_diagonal_sign(D, 43)
    g = torch.Generator(device="cuda")
    g.manual_seed(4)
    kp, kn = encoded_kv_on_gpu(tq, g, n_kv, total, bits, dev(ks))
    vp, vn = encoded_kv_on_gpu(tq, g, n_kv, total, bits, dev(vs))
    q = rng.standard_normal((n_seq, n_kv * n_rep, D)).astype(np.float16).astype(F32)
    sc = 1 / math.sqrt(D)
    q_rot = tq.prerotate_query(dev(q.reshape(-1, D)), dev(ks)).reshape(n_seq, n_kv * n_rep, D)
    kw = dict(n_rep=n_rep, seq_offsets=dev(offs), max_seq_len=max_len)
    a = tq.flash_decode(q_rot, kp, kn, vp, vn, c, c, dev(vs), D, bits, sc, out_dtype=torch.float16, **kw)
    zero_mask = torch.zeros((n_seq, 1, max_len), device="cuda")
    t = tq.flash_decode(q_rot, kp, kn, vp, vn, c, c, dev(vs), D, bits, sc, out_dtype=torch.float16, mask=zero_mask, **kw)
    f = tq.flash_decode(q_rot, kp, kn, vp, vn, c, c, dev(vs), D, bits, sc, precision="fp32", **kw)
    assert a.dtype == torch.float16
    a, t, f = host(a).astype(F32), host(t).astype(F32), host(f)
    close(a.reshape(-1, D), f.reshape(-1, D), rel=2.5e-3, abs_=1e-4, row_scale=True)     # 2e-3 + fp16 rounding of the output
    close(t.reshape(-1, D), f.reshape(-1, D), rel=2.5e-3, abs_=1e-4, row_scale=True)
    close(a.reshape(-1, D), t.reshape(-1, D), rel=2e-3, abs_=1e-4, row_scale=True)
    hk, hkn, hv, hvn = host(kp), host(kn), host(vp), host(vn)
    order = np.argsort(lens)
    for i in (order[0], order[1], order[-1]):
        s0, s1 = offs[i], offs[i + 1]
        want = o.flash_attention_turboquant(o.prerotate_query(q[i], ks), hk[:, s0:s1], hkn[:, s0:s1], hv[:, s0:s1],
                                            hvn[:, s0:s1], c, c, vs, D, bits, sc, 16, n_rep)
        close(a[i], want, rel=2.5e-3, abs_=1e-4, row_scale=True)
        close(f[i], want, abs_=1e-4, row_scale=True)               # the float32 kernels: no fp16 anywhere


def test_config5_full_size_encode_paths_agree(tq):
    """benchmark configuration 5, encode half, at full size: 1 048 576 fp16 vectors with one channel scaled
    x20.  The streaming encoder (rows in multiples of 16) and the generic one-wavefront-per-vector encoder
    (taken for a row count that is not a multiple of 16) must produce identical words and norms over the
    whole tensor; 32 768 vectors spread over it are also compared with the oracle bit for bit."""
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    n = 131072 * 8
    x = torch.randn((n, 128), generator=g, device="cuda", dtype=torch.float16)
    x[:, 17] *= 20
    c, b = tables(3)
    s = o.random_diagonal_sign(128, 42)
    fp, fn = tq.fused_quantize(x, dev(s), b, 128, 3)                    # streaming kernel
    gp, gn = tq.fused_quantize(x[: n - 1], dev(s), b, 128, 3)           # generic kernel: n - 1 rows
    assert torch.equal(fp[: n - 1].view(torch.int32), gp.view(torch.int32)) and torch.equal(fn[: n - 1], gn)
    pick = torch.arange(0, n, 32, device="cuda")
    wp, wn = o.fused_quantize(host(x[pick]), s, b, 128, 3)
    assert np.array_equal(host(fp.view(torch.int32)[pick]).view(np.uint32), wp) and np.array_equal(host(fn[pick]), wn)


def test_config5_full_size_prefill_rows_are_decode_steps(tq):
    """benchmark configuration 5, attention half, at full size: a 512-row causal chunk at the end of a 131 072-position
    packed cache, 32 q / 8 kv heads.  Row i of the chunk is one decode step over positions 0 .. T-512+i: three
    rows are compared with the float32 flash-decode kernels (a separate code path) over those prefixes, and with
    the ORACLE's flash attention over the same prefixes -- the last row (all 131 072 positions) on kv heads 0 and 7,
    the first and the middle row on kv head 3 (the float64 oracle takes ~8 s per kv head at this length)."""
    g = torch.Generator(device="cuda")
    g.manual_seed(55)
    n_kv, n_rep, T, n_rows, D, bits = 8, 4, 131072, 512, 128, 3
    c, b = tables(bits)
    ks, vs = dev(o.random_diagonal_sign(D, 42)), dev(o.random_diagonal_sign(D, 43))
    # the configuration's data: N(0,1) fp16 rows with 1 % of the channels (one of 128, drawn from the seed) scaled x20
    ch = int(torch.randint(0, D, (1,), generator=g, device="cuda").item())
    kp, kn = encoded_kv_on_gpu(tq, g, n_kv, T, bits, ks, outlier_channel=ch)
    vp, vn = encoded_kv_on_gpu(tq, g, n_kv, T, bits, vs, outlier_channel=ch)
    q = torch.randn((n_kv * n_rep, n_rows, D), generator=g, device="cuda", dtype=torch.float16)
    sc = 1 / math.sqrt(D)
    got = tq.prefill_attention(q, kp, kn, vp, vn, c, c, ks, vs, D, bits, sc, n_rep=n_rep, out_dtype=torch.float32)
    for i in (0, 255, 511):
        L = T - n_rows + i + 1
        q_rot = tq.prerotate_query(q[:, i].float(), ks)
        ref = tq.flash_attention_turboquant(q_rot, kp[:, :L], kn[:, :L], vp[:, :L], vn[:, :L], c, c, vs, D, bits, sc,
                                            n_rep=n_rep, precision="fp32")
        close(host(got[:, i]), host(ref), row_scale=True)
    hks = o.random_diagonal_sign(D, 42)
    hvs = o.random_diagonal_sign(D, 43)
    for i, heads in ((511, (0, 7)), (0, (3,)), (255, (3,))):
        L = T - n_rows + i + 1
        for h in heads:
            qh = host(q[h * n_rep:(h + 1) * n_rep, i]).astype(F32)
            want = o.flash_attention_turboquant(o.prerotate_query(qh, hks), host(kp[h:h + 1, :L]), host(kn[h:h + 1, :L]),
                                                host(vp[h:h + 1, :L]), host(vn[h:h + 1, :L]), c, c, hvs, D, bits, sc, 16, n_rep)
            close(host(got[h * n_rep:(h + 1) * n_rep, i]), want, row_scale=True)


def test_config3_full_size_scores(tq):
    """benchmark configuration 3 at its largest size: 28 q / 4 kv heads against 65 536 packed keys; the float32
    kernel to float32 rounding and the matrix-core kernel to 1e-3 of the row scale, both against the oracle."""
    rng = np.random.default_rng(3)
    n_kv, n_rep, T, D, bits = 4, 7, 65536, 128, 3
    c, b = tables(bits)
    ks = o.random_diagonal_sign(D, 42)
    kp = o.pack_indices(rng.integers(0, 8, size=(n_kv, T, D)).astype(np.uint8), bits)
    kn = (rng.random((n_kv, T)) * 8 + 7).astype(F32)
    q_rot = o.prerotate_query(rng.standard_normal((n_kv * n_rep, D)).astype(F32), ks)
    want = o.prerot_fused_qk_scores(q_rot, kp, kn, c, D, bits, n_rep)
    got32 = host(tq.prerot_fused_qk_scores(dev(q_rot), dev(kp), dev(kn), c, D, bits, n_rep))
    close(got32, want, rel=1e-5, abs_=1e-4)
    got16 = host(tq.prerot_fused_qk_scores(dev(q_rot), dev(kp), dev(kn), c, D, bits, n_rep, precision="fp16"))
    close(got16, want, rel=1e-3, abs_=1e-3 * float(np.abs(want).max()))


def test_vonly_decode_bf16_queries_take_the_matrix_core_path(tq):
    """bf16 queries (a bf16 model over an fp16 key cache): converted to fp16 on load, which is exact for
    query-sized values, so the result must match the oracle evaluated on the bf16 values, for the tile
    pass (T = 2048) and the streaming pass (T = 16384, 4 kv heads x 8 heads each)."""
    rng = np.random.default_rng(81)
    D, bits, sc = 128, 3, 1 / math.sqrt(128)
    for n_kv, n_rep, T in ((4, 7, 2048), (4, 8, 16384)):
        c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, T, D, bits)
        qt = torch.from_numpy(rng.standard_normal((1, n_kv * n_rep, D)).astype(F32)).to(torch.bfloat16)
        got = tq.vonly_decode(qt.cuda(), dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc, n_rep=n_rep,
                              out_dtype=torch.bfloat16)
        assert got.dtype == torch.bfloat16
        want = o.vonly_decode_attention(qt[0].float().numpy(), K, vp, vn, c, vs, D, bits, sc)
        err = np.abs(got[0].float().cpu().numpy().astype(np.float64) - want)
        assert (err <= 1e-3 + 6e-3 * np.abs(want)).all(), err.max()       # bf16 rounding of the output: 2^-8
        got32 = host(tq.vonly_decode(qt.cuda(), dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc, n_rep=n_rep))
        close(got32[0], want)


def test_vonly_decode_float32_queries_keep_their_precision(tq):
    """float32 queries on the matrix-core path enter as fp16 value + fp16 remainder.  On data with x20 outlier
    channels in K (peaked softmax, logits in the hundreds) rounding the query to one fp16 shows; the
    two-term form must stay close to the float32 kernels."""
    rng = np.random.default_rng(91)
    n_kv, n_rep, T, D, bits = 4, 7, 4096, 128, 3
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, T, D, bits, outliers=True)
    q = rng.standard_normal((1, n_kv * n_rep, D)).astype(F32)
    q[..., 7] *= 3
    sc = 1 / math.sqrt(D)
    args = (dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc)
    ref = host(tq.vonly_decode(dev(q), *args, n_rep=n_rep, precision="fp32"))[0]
    two = host(tq.vonly_decode(dev(q), *args, n_rep=n_rep))[0]
    one = host(tq.vonly_decode(dev(q.astype(np.float16)), *args, n_rep=n_rep))[0]
    scale = np.abs(ref).max(axis=-1, keepdims=True)
    e_two, e_one = (np.abs(two - ref) / scale).max(), (np.abs(one - ref) / scale).max()
    print(f"max error / row scale: two-term {e_two:.2e}, one fp16 {e_one:.2e}")
    assert e_two < 1e-3 and e_two < 0.5 * e_one
    want = o.vonly_decode_attention(q[0], K, vp, vn, c, vs, D, bits, sc)
    close(two, want, row_scale=True)


def test_encode_overflowing_norm_and_infinite_elements(tq):
    """float32 vectors whose sum of squares overflows (norm = inf: every finite element divides to 0, index 3)
    and vectors with an infinite element (inf / inf = NaN spreads to every output, index 0): the streaming
    and the generic encoder must both follow the oracle."""
    rng = np.random.default_rng(92)
    c, b = tables(3)
    s = o.random_diagonal_sign(128, 42)
    x = rng.standard_normal((48, 128)).astype(F32)
    x[3] *= 1e25
    x[7, 11] = np.inf
    x[20, 5] = -np.inf
    x[21] *= 3e19
    with np.errstate(all="ignore"):
        wp, wn = o.fused_quantize(x, s, b, 128, 3)
    for rows in (48, 47):                                              # streaming / generic kernel
        gp, gn = tq.fused_quantize(dev(x[:rows]), dev(s), b, 128, 3)
        assert np.array_equal(host(gp), wp[:rows])
        assert np.array_equal(host(gn), wn[:rows], equal_nan=True)
    assert np.isinf(wn[3]) and (o.unpack_indices(wp[3:4], 3, 128) == 3).all()
    assert (o.unpack_indices(wp[7:8], 3, 128) == 0).all()


@pytest.mark.parametrize("scale", [1e-19, 1e-21, 1e-22, 1e-23, 1e-30, 1e-42])
def test_encode_tiny_float32_inputs(tq, scale):
    """float32 inputs whose squares are subnormal or underflow (norm subnormal or 0, clamped to 1e-8 by the
    quantiser): both encoders must follow the oracle bit for bit, subnormal arithmetic included."""
    rng = np.random.default_rng(93)
    c, b = tables(3)
    s = o.random_diagonal_sign(128, 42)
    x = (rng.standard_normal((48, 128)) * scale).astype(F32)
    wp, wn = o.fused_quantize(x, s, b, 128, 3)
    for rows in (48, 47):                                              # streaming / generic kernel
        gp, gn = tq.fused_quantize(dev(x[:rows]), dev(s), b, 128, 3)
        assert np.array_equal(host(gp), wp[:rows]) and np.array_equal(host(gn), wn[:rows])


def test_fully_masked_rows_yield_zeros(tq):
    """A query head whose every position is masked: the kernels return zeros for it (softmax over an empty set;
    the reference's mx.softmax would give NaN there) and leave the other heads untouched, on the matrix-core
    and the float32 paths of both fused decode ops."""
    rng = np.random.default_rng(94)
    n_kv, n_rep, T, D, bits = 2, 4, 700, 128, 3
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, T, D, bits)
    q = rng.standard_normal((1, n_kv * n_rep, D)).astype(np.float16)
    sc = 1 / math.sqrt(D)
    mask = np.zeros((1, n_kv * n_rep, T), F32)
    mask[0, 0, :] = -np.inf                       # head 0 sees nothing
    mask[0, 5, 100:] = -np.inf                    # head 5 sees the first 100 positions
    q_rot = tq.prerotate_query(dev(q.reshape(-1, D).astype(F32)), dev(ks)).reshape(1, -1, D)
    for precision in ("fp16", "fp32"):
        a = host(tq.vonly_decode(dev(q), dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc, n_rep=n_rep,
                                 mask=dev(mask), precision=precision))[0]
        f = host(tq.flash_decode(q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, sc, n_rep=n_rep,
                                 mask=dev(mask), precision=precision))[0]
        assert (a[0] == 0).all() and (f[0] == 0).all(), precision
        want_v = o.vonly_decode_attention(q[0, 4:8], K[1:], vp[1:], vn[1:], c, vs, D, bits, sc, mask=mask[0, 4:8])
        close(a[4:8], want_v)
        want_f = o.turboquant_attention_single(q[0, 4:8].astype(F32), kp[1:], kn[1:], vp[1:], vn[1:], c, ks, c, vs,
                                               D, bits, sc, mask=mask[0, 4:8])
        close(f[4:8], want_f)


@pytest.mark.parametrize("n_rows,T,mask_kind", [(1, 1, "none"), (3, 7, "row"), (28, 4096, "shared"), (28, 32770, "none"),
                                                (2, 65536, "row"), (7, 16384, "shared"), (300, 513, "row"), (28, 32768, "none")])
def test_softmax_rows_shapes(tq, n_rows, T, mask_kind):
    """softmax_rows (fused_attention.py:78-94) on few long rows (several workgroups per row), many short rows,
    lengths that are not a multiple of 4, with a shared or a per-row additive mask: against float64 numpy."""
    rng = np.random.default_rng(n_rows * 1000 + T)
    x = (rng.standard_normal((n_rows, T)) * 3).astype(F32)
    scale = 0.37
    mask = None
    if mask_kind != "none":
        shape = (T,) if mask_kind == "shared" else (n_rows, T)
        mask = np.where(rng.random(shape) < 0.3, -np.inf, 0.0).astype(F32)
        mask[..., 0] = 0.0
    got = host(tq.softmax_rows(dev(x), scale, None if mask is None else dev(mask)))
    z = x.astype(np.float64) * np.float64(F32(scale)) + (0.0 if mask is None else mask.astype(np.float64))
    z = z - z.max(axis=-1, keepdims=True)
    want = np.exp(z) / np.exp(z).sum(axis=-1, keepdims=True)
    assert got.shape == want.shape
    assert np.abs(got - want).max() <= 1e-7 + 2e-6 * want.max()
    assert np.abs(got.sum(axis=-1) - 1.0).max() < 1e-5


# ------------------------------------------------------------------ thresholded V-only decode in one call

@pytest.mark.parametrize("n_seq,n_kv,n_rep,T,thr,qdt,mask_kind", [
    (1, 4, 7, 1500, 1e-5, np.float16, "none"), (2, 2, 4, 513, 1e-3, np.float32, "seq"),
    (1, 8, 1, 2048, 1e-4, np.float16, "head"), (3, 1, 16, 77, 1e-2, np.float16, "none"),
    (1, 4, 7, 4099, 1e-5, np.float32, "head"), (2, 3, 5, 1, 1e-5, np.float16, "none"),
    # more than 128 statistics per kv head: the weights pass folds them in more than one sweep
    (1, 2, 7, 40001, 1e-5, np.float16, "none"), (1, 1, 4, 70000, 1e-6, np.float32, "none"),
    # more than 1024 steps of 256 positions in all: the weights pass in its streaming form
    (4, 8, 2, 9001, 1e-5, np.float16, "none"), (6, 8, 1, 6000, 1e-4, np.float32, "head")])
def test_vonly_sparse_decode_matches_oracle(tq, n_seq, n_kv, n_rep, T, thr, qdt, mask_kind):
    """tq_vonly_sparse_decode_attn (scores pass, weights-and-values pass, merge) against the oracle's
    dense scores -> softmax -> thresholded value sum, cache layout with an allocation longer than the
    valid length."""
    rng = np.random.default_rng(7 * T + n_rep)
    D, bits, sc = 128, 3, 1 / math.sqrt(128)
    n_q = n_kv * n_rep
    T_alloc = T + 37
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_seq * n_kv, T_alloc, D, bits)
    K, vp, vn = (a.reshape(n_seq, n_kv, *a.shape[1:]) for a in (K, vp, vn))
    q = rng.standard_normal((n_seq, n_q, D)).astype(qdt)
    mask = _draw_mask(rng, mask_kind, n_seq, n_q, T)
    kw = {} if mask is None else dict(mask=dev(mask))
    got = host(tq.vonly_decode(dev(q), dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc, n_rep=n_rep, seq_len=T,
                               sparse_v_threshold=thr, **kw))
    dropped = 0
    for i in range(n_seq):
        mi = None if mask is None else np.broadcast_to(mask[i], (n_q, T))
        want = o.vonly_decode_attention(q[i], K[i, :, :T], vp[i, :, :T], vn[i, :, :T], c, vs, D, bits, sc,
                                        threshold=thr, mask=mi)
        dense = o.vonly_decode_attention(q[i], K[i, :, :T], vp[i, :, :T], vn[i, :, :T], c, vs, D, bits, sc, mask=mi)
        dropped += int(np.abs(want - dense).max() > 0)
        close(got[i], want)
    if T >= 500:
        assert dropped > 0                         # the threshold did remove something in these cases


def test_vonly_sparse_decode_ragged_batch_and_dtypes(tq):
    """Ragged batch (sequence offsets into [n_kv, sum(L), *] tensors, lengths that end inside a tile and inside
    a wave's rows), bf16 queries and fp16 output."""
    rng = np.random.default_rng(401)
    n_kv, n_rep, D, bits, sc, thr = 4, 7, 128, 3, 1 / math.sqrt(128), 1e-4
    lens = np.array([1300, 1, 512, 65, 2049])
    offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, int(offs[-1]), D, bits)
    qt = torch.from_numpy(rng.standard_normal((len(lens), n_kv * n_rep, D)).astype(F32)).to(torch.bfloat16)
    got = tq.vonly_decode(qt.cuda(), dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc, n_rep=n_rep,
                          seq_offsets=dev(offs), max_seq_len=int(lens.max()), out_dtype=torch.float16,
                          sparse_v_threshold=thr)
    assert got.dtype == torch.float16
    got = host(got.float())
    for i in range(len(lens)):
        a, e = offs[i], offs[i + 1]
        want = o.vonly_decode_attention(qt[i].float().numpy(), K[:, a:e], vp[:, a:e], vn[:, a:e], c, vs, D, bits, sc,
                                        threshold=thr)
        close(got[i], want, rel=3e-3, abs_=2e-3)           # + fp16 rounding of the output


def test_vonly_sparse_decode_threshold_limits(tq):
    """A threshold above every weight drops every position (exact zeros, sparse_v.py:59-65); a threshold below
    every representable weight changes nothing against the dense fused step; a fully masked head yields zeros."""
    rng = np.random.default_rng(402)
    n_kv, n_rep, T, D, bits, sc = 2, 4, 900, 128, 3, 1 / math.sqrt(128)
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, T, D, bits)
    q = rng.standard_normal((1, n_kv * n_rep, D)).astype(np.float16)
    args = (dev(q), dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc)
    none_left = host(tq.vonly_decode(*args, n_rep=n_rep, sparse_v_threshold=2.0))
    assert (none_left == 0).all()
    all_kept = host(tq.vonly_decode(*args, n_rep=n_rep, sparse_v_threshold=1e-37))
    dense = host(tq.vonly_decode(*args, n_rep=n_rep))
    close(all_kept, dense, rel=1e-3, abs_=2e-4)
    close(all_kept[0], o.vonly_decode_attention(q[0], K, vp, vn, c, vs, D, bits, sc))
    mask = np.zeros((1, n_kv * n_rep, T), F32)
    mask[0, 2, :] = -np.inf
    masked = host(tq.vonly_decode(*args, n_rep=n_rep, mask=dev(mask), sparse_v_threshold=1e-5))[0]
    assert (masked[2] == 0).all()
    close(masked[4:], o.vonly_decode_attention(q[0, 4:], K[1:], vp[1:], vn[1:], c, vs, D, bits, sc, threshold=1e-5))


def test_vonly_sparse_decode_rejects_other_shapes(tq):
    """dim 64 caches have no one-call thresholded step: the wrapper says which ops to compose."""
    rng = np.random.default_rng(403)
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, 2, 64, 64, 4)
    q = rng.standard_normal((1, 2, 64)).astype(np.float16)
    with pytest.raises(ValueError, match="compose dense_qk_scores"):
        tq.vonly_decode(dev(q), dev(K), dev(vp), dev(vn), c, dev(vs), 64, 4, 0.125, n_rep=1, sparse_v_threshold=1e-5)


@pytest.mark.parametrize("seed", range(12))
def test_decode_sweep_vonly_sparse(tq, seed):
    """The thresholded step on the drawn decode shapes (ragged and cache-layout batches, masks, query dtypes)."""
    rng, n_kv, n_rep, ragged, n_seq, lens, mask_kind, qdt = _draw_decode_case(500 + seed)
    D, bits, sc = 128, 3, 1 / math.sqrt(128)
    n_q = n_kv * n_rep
    thr = float(rng.choice([1e-5, 1e-4, 1e-3]))
    print(f"seed {seed}: n_kv {n_kv} n_rep {n_rep} ragged {ragged} lens {lens.tolist()} mask {mask_kind} "
          f"q {np.dtype(qdt).name} thr {thr:g}", flush=True)
    q = rng.standard_normal((n_seq, n_q, D)).astype(qdt)
    if ragged:
        offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, int(offs[-1]), D, bits)
        kw = dict(seq_offsets=dev(offs), max_seq_len=int(lens.max()))
        per_seq = [tuple(a[:, offs[i]:offs[i + 1]] for a in (K, vp, vn)) for i in range(n_seq)]
        mask = None
    else:
        T = int(lens[0])
        T_alloc = T + int(rng.integers(0, 70))
        c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_seq * n_kv, T_alloc, D, bits)
        K, vp, vn = (a.reshape(n_seq, n_kv, *a.shape[1:]) for a in (K, vp, vn))
        kw = dict(seq_len=T)
        per_seq = [tuple(a[i, :, :T] for a in (K, vp, vn)) for i in range(n_seq)]
        mask = _draw_mask(rng, mask_kind, n_seq, n_q, T)
        if mask is not None:
            kw["mask"] = dev(mask)
    got = host(tq.vonly_decode(dev(q), dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc, n_rep=n_rep,
                               sparse_v_threshold=thr, **kw))
    for i in range(n_seq):
        Ki, vpi, vni = per_seq[i]
        mi = None if mask is None else np.broadcast_to(mask[i], (n_q, mask.shape[-1]))
        close(got[i], o.vonly_decode_attention(q[i], Ki, vpi, vni, c, vs, D, bits, sc, threshold=thr, mask=mi))


# ------------------------------------------------------------------ thresholded decode over packed keys in one call

def _packed_weights(q, kp, kn, c, ks, sc, n_rep, mask):
    """Final softmax weights of one sequence over packed keys, as the oracle's turboquant_attention forms them."""
    s = o.prerot_fused_qk_scores(o.prerotate_query(q, ks), kp, kn, c, 128, 3, n_rep) * F32(sc)
    if mask is not None:
        s = s + np.asarray(mask, dtype=F32)
    return o._softmax64(s).astype(F32)


@pytest.mark.parametrize("n_seq,n_kv,n_rep,T,thr,mask_kind", [
    (1, 8, 4, 1500, 1e-5, "none"), (2, 2, 7, 513, 1e-3, "seq"), (1, 4, 1, 2048, 1e-4, "head"),
    (3, 1, 16, 77, 1e-2, "none"), (2, 3, 5, 1, 1e-5, "none"),
    # more than 128 tiles per kv head: the weights pass folds the statistics in more than one sweep
    (1, 1, 4, 70001, 1e-6, "none"),
    # masked and large: scores by the tile pass, weights and values by the streaming pass
    (4, 8, 2, 9001, 1e-5, "head")])
def test_flash_sparse_decode_matches_oracle(tq, n_seq, n_kv, n_rep, T, thr, mask_kind):
    """tq_flash_sparse_decode against the oracle's turboquant_attention with a sparse-V threshold
    (scores of packed K -> scale, mask, softmax -> thresholded value sum)."""
    rng = np.random.default_rng(11 * T + n_rep)
    D, bits, sc = 128, 3, 1 / math.sqrt(128)
    n_q = n_kv * n_rep
    T_alloc = T + 21
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_seq * n_kv, T_alloc, D, bits)
    kp, kn, vp, vn = (a.reshape(n_seq, n_kv, *a.shape[1:]) for a in (kp, kn, vp, vn))
    q = rng.standard_normal((n_seq, n_q, D)).astype(F32)
    mask = _draw_mask(rng, mask_kind, n_seq, n_q, T)
    kw = {} if mask is None else dict(mask=dev(mask))
    q_rot = tq.prerotate_query(dev(q.reshape(-1, D)), dev(ks)).reshape(n_seq, n_q, D)
    got = host(tq.flash_decode(q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, sc, n_rep=n_rep,
                               seq_len=T, sparse_v_threshold=thr, **kw))
    for i in range(n_seq):
        mi = None if mask is None else np.broadcast_to(mask[i], (n_q, T))
        want = o.turboquant_attention_single(q[i], kp[i, :, :T], kn[i, :, :T], vp[i, :, :T], vn[i, :, :T], c, ks, c, vs,
                                             D, bits, sc, sparse_v_threshold=thr, mask=mi)
        w = _packed_weights(q[i], kp[i, :, :T], kn[i, :, :T], c, ks, sc, n_rep, mi)
        close(got[i], want, extra=threshold_slack(w, thr, vp[i, :, :T], vn[i, :, :T], c, vs, n_rep, 3e-3))


def test_flash_sparse_decode_ragged_and_limits(tq):
    """Ragged batch; a threshold above every weight gives exact zeros; a vanishing one equals the dense fused step."""
    rng = np.random.default_rng(411)
    n_kv, n_rep, D, bits, sc = 8, 4, 128, 3, 1 / math.sqrt(128)
    lens = np.array([1300, 1, 512, 65, 2049])
    offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, int(offs[-1]), D, bits)
    q = rng.standard_normal((len(lens), n_kv * n_rep, D)).astype(F32)
    q_rot = tq.prerotate_query(dev(q.reshape(-1, D)), dev(ks)).reshape(len(lens), -1, D)
    args = (q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, sc)
    kw = dict(n_rep=n_rep, seq_offsets=dev(offs), max_seq_len=int(lens.max()))
    got = host(tq.flash_decode(*args, sparse_v_threshold=1e-4, **kw))
    for i in range(len(lens)):
        a, e = offs[i], offs[i + 1]
        want = o.turboquant_attention_single(q[i], kp[:, a:e], kn[:, a:e], vp[:, a:e], vn[:, a:e], c, ks, c, vs,
                                             D, bits, sc, sparse_v_threshold=1e-4)
        w = _packed_weights(q[i], kp[:, a:e], kn[:, a:e], c, ks, sc, n_rep, None)
        close(got[i], want, extra=threshold_slack(w, 1e-4, vp[:, a:e], vn[:, a:e], c, vs, n_rep, 3e-3))
    assert (host(tq.flash_decode(*args, sparse_v_threshold=2.0, **kw)) == 0).all()
    close(host(tq.flash_decode(*args, sparse_v_threshold=1e-37, **kw)), host(tq.flash_decode(*args, **kw)),
          rel=1e-3, abs_=2e-4)
    with pytest.raises(ValueError, match="compose prerot_fused_qk_scores"):
        c4, ks4, vs4, K4, V4, kp4, kn4, vp4, vn4 = kv_fixture(rng, 2, 64, 64, 4)
        tq.flash_decode(torch.zeros((1, 2, 64), device="cuda"), dev(kp4), dev(kn4), dev(vp4), dev(vn4), c4, c4, dev(vs4),
                        64, 4, 0.125, n_rep=1, sparse_v_threshold=1e-5)


def test_flash_sparse_decode_streaming_scores_pass(tq):
    """Calls large enough for the streaming form of the scores pass (one statistics entry per workgroup range of several
    256-position steps): a ragged batch whose sequences start at every misalignment of the 52-byte rows and end inside
    a step, inside a wave's rows and one row past a step; and a cache layout with an allocation longer than the length."""
    rng = np.random.default_rng(413)
    n_kv, n_rep, D, bits, sc, thr = 8, 4, 128, 3, 1 / math.sqrt(128), 1e-5
    lens = np.array([4097, 2561, 1025, 7000, 1, 3333, 5121, 6143])
    n_seq = len(lens)
    assert _flash_plan(tq, n_seq, n_kv, int(lens.max()), True) >= 2
    offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, int(offs[-1]), D, bits)
    q = rng.standard_normal((n_seq, n_kv * n_rep, D)).astype(F32)
    q_rot = tq.prerotate_query(dev(q.reshape(-1, D)), dev(ks)).reshape(n_seq, -1, D)
    got = host(tq.flash_decode(q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, sc, n_rep=n_rep,
                               seq_offsets=dev(offs), max_seq_len=int(lens.max()), sparse_v_threshold=thr))
    dropped = 0
    for i in range(n_seq):
        a, e = offs[i], offs[i + 1]
        want = o.turboquant_attention_single(q[i], kp[:, a:e], kn[:, a:e], vp[:, a:e], vn[:, a:e], c, ks, c, vs,
                                             D, bits, sc, sparse_v_threshold=thr)
        dense = o.turboquant_attention_single(q[i], kp[:, a:e], kn[:, a:e], vp[:, a:e], vn[:, a:e], c, ks, c, vs, D, bits, sc)
        dropped += int(np.abs(want - dense).max() > 0)
        w = _packed_weights(q[i], kp[:, a:e], kn[:, a:e], c, ks, sc, n_rep, None)
        close(got[i], want, extra=threshold_slack(w, thr, vp[:, a:e], vn[:, a:e], c, vs, n_rep, 3e-3))
    assert dropped >= 4                                      # the threshold removed something in the long sequences
    # cache layout, two sequences of 9001 positions in an allocation of 9030
    T, T_alloc = 9001, 9030
    assert _flash_plan(tq, 2, n_kv, T, False) >= 2
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, 2 * n_kv, T_alloc, D, bits)
    kp, kn, vp, vn = (x.reshape(2, n_kv, *x.shape[1:]) for x in (kp, kn, vp, vn))
    q = rng.standard_normal((2, n_kv * n_rep, D)).astype(F32)
    q_rot = tq.prerotate_query(dev(q.reshape(-1, D)), dev(ks)).reshape(2, -1, D)
    got = host(tq.flash_decode(q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, sc, n_rep=n_rep,
                               seq_len=T, sparse_v_threshold=thr))
    for i in range(2):
        want = o.turboquant_attention_single(q[i], kp[i, :, :T], kn[i, :, :T], vp[i, :, :T], vn[i, :, :T], c, ks, c, vs,
                                             D, bits, sc, sparse_v_threshold=thr)
        w = _packed_weights(q[i], kp[i, :, :T], kn[i, :, :T], c, ks, sc, n_rep, None)
        close(got[i], want, extra=threshold_slack(w, thr, vp[i, :, :T], vn[i, :, :T], c, vs, n_rep, 3e-3))


@pytest.mark.parametrize("seed", range(12))
def test_decode_sweep_flash_sparse(tq, seed):
    """The thresholded packed-key step on the drawn decode shapes."""
    rng, n_kv, n_rep, ragged, n_seq, lens, mask_kind, qdt = _draw_decode_case(600 + seed)
    D, bits, sc = 128, 3, 1 / math.sqrt(128)
    n_q = n_kv * n_rep
    thr = float(rng.choice([1e-5, 1e-4, 1e-3]))
    print(f"seed {seed}: n_kv {n_kv} n_rep {n_rep} ragged {ragged} lens {lens.tolist()} mask {mask_kind} thr {thr:g}", flush=True)
    q = rng.standard_normal((n_seq, n_q, D)).astype(F32)
    if ragged:
        offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, int(offs[-1]), D, bits)
        kw = dict(seq_offsets=dev(offs), max_seq_len=int(lens.max()))
        per_seq = [tuple(a[:, offs[i]:offs[i + 1]] for a in (kp, kn, vp, vn)) for i in range(n_seq)]
        mask = None
    else:
        T = int(lens[0])
        T_alloc = T + int(rng.integers(0, 70))
        c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_seq * n_kv, T_alloc, D, bits)
        kp, kn, vp, vn = (a.reshape(n_seq, n_kv, *a.shape[1:]) for a in (kp, kn, vp, vn))
        kw = dict(seq_len=T)
        per_seq = [tuple(a[i, :, :T] for a in (kp, kn, vp, vn)) for i in range(n_seq)]
        mask = _draw_mask(rng, mask_kind, n_seq, n_q, T)
        if mask is not None:
            kw["mask"] = dev(mask)
    q_rot = tq.prerotate_query(dev(q.reshape(-1, D)), dev(ks)).reshape(n_seq, n_q, D)
    got = host(tq.flash_decode(q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, sc, n_rep=n_rep,
                               sparse_v_threshold=thr, **kw))
    for i in range(n_seq):
        kpi, kni, vpi, vni = per_seq[i]
        mi = None if mask is None else np.broadcast_to(mask[i], (n_q, mask.shape[-1]))
        w = _packed_weights(q[i], kpi, kni, c, ks, sc, n_rep, mi)
        close(got[i], o.turboquant_attention_single(q[i], kpi, kni, vpi, vni, c, ks, c, vs, D, bits, sc,
                                                    sparse_v_threshold=thr, mask=mi),
              extra=threshold_slack(w, thr, vpi, vni, c, vs, n_rep, 3e-3))


# ------------------------------------------------------------------ decode step from the query itself (rotation in-kernel)

@pytest.mark.parametrize("qdt", ["float32", "float16", "bfloat16"])
@pytest.mark.parametrize("case", ["tile", "stream_ragged", "masked", "threshold"])
def test_flash_decode_from_q_equals_prerotate_then_flash(tq, qdt, case):
    """tq_flash_decode_from_q rotates the query inside the attention kernels with the stage order of
    tq_prerotate_query: the result must be IDENTICAL to prerotate_query followed by flash_decode, for every
    query dtype, on the tile pass, the streaming pass (ragged batch), with a mask and with a threshold."""
    rng = np.random.default_rng(sum(map(ord, qdt + case)))
    D, bits, sc = 128, 3, 1 / math.sqrt(128)
    n_kv, n_rep = (8, 4) if case == "stream_ragged" else (4, 7)
    n_q = n_kv * n_rep
    c, b = tables(bits)
    ks, vs = o.random_diagonal_sign(D, 42), o.random_diagonal_sign(D, 43)
    kw = {}
    if case == "stream_ragged":
        lens = np.array([4097, 2561, 1025, 7000, 1, 3333, 5121, 6143])
        offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        assert _flash_plan(tq, len(lens), n_kv, int(lens.max()), True) >= 2
        shape, n_seq = (n_kv, int(offs[-1])), len(lens)
        kw = dict(seq_offsets=dev(offs), max_seq_len=int(lens.max()))
    else:
        n_seq, T = 2, 1111
        shape = (n_seq, n_kv, T + 13)
        kw = dict(seq_len=T)
        if case == "masked":
            kw["mask"] = dev(_draw_mask(rng, "head", n_seq, n_q, T))
        if case == "threshold":
            kw["sparse_v_threshold"] = 1e-4
    kp = o.pack_indices(rng.integers(0, 8, size=shape + (D,)).astype(np.uint8), bits)
    vp = o.pack_indices(rng.integers(0, 8, size=shape + (D,)).astype(np.uint8), bits)
    kn = (rng.random(shape) * 12 + 6).astype(F32)
    vn = (rng.random(shape) + 0.5).astype(F32)
    q = torch.from_numpy(rng.standard_normal((n_seq, n_q, D)).astype(F32)).to(getattr(torch, qdt)).cuda()
    q_rot = tq.prerotate_query(q.reshape(-1, D), dev(ks)).reshape(n_seq, n_q, D)
    two = tq.flash_decode(q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, sc, n_rep=n_rep, **kw)
    one = tq.flash_decode_from_q(q, dev(ks), dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, sc, n_rep=n_rep, **kw)
    assert torch.equal(one, two)
    assert torch.isfinite(one).all()


def test_flash_decode_from_q_against_oracle_and_shape_limits(tq):
    rng = np.random.default_rng(77)
    n_kv, n_rep, T, D, bits, sc = 2, 16, 700, 128, 3, 1 / math.sqrt(128)
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, n_kv, T, D, bits)
    q = rng.standard_normal((1, n_kv * n_rep, D)).astype(np.float16)
    got = host(tq.flash_decode_from_q(dev(q), dev(ks), dev(kp[None]), dev(kn[None]), dev(vp[None]), dev(vn[None]), c, c,
                                      dev(vs), D, bits, sc, n_rep=n_rep))
    close(got[0], o.turboquant_attention_single(q[0].astype(F32), kp, kn, vp, vn, c, ks, c, vs, D, bits, sc))
    c4, ks4, vs4, K4, V4, kp4, kn4, vp4, vn4 = kv_fixture(rng, 2, 64, 64, 4)
    with pytest.raises(ValueError, match="prerotate_query"):
        tq.flash_decode_from_q(torch.zeros((1, 2, 64), device="cuda"), dev(ks4), dev(kp4[None]), dev(kn4[None]),
                               dev(vp4[None]), dev(vn4[None]), c4, c4, dev(vs4), 64, 4, 0.125, n_rep=1)


# ------------------------------------------------------------------ tensors with more than 2^31 elements / words

def test_addressing_past_2g_elements(tq):
    """Tensors whose element (encode input, dequant output, fp16 keys) or word (packed rows) count exceeds 2^31:
    every address in the kernels must be formed in 64 bits.  Data are generated on the GPU; rows at the start,
    in the middle and at the very end are checked against the oracle (encode / dequant bit for bit), and a short
    sequence stored BEHIND a very long one in a ragged batch is attended through both fused decode steps."""
    D, bits, sc = 128, 3, 1 / math.sqrt(128)
    c, b = tables(bits)
    ks, vs = o.random_diagonal_sign(D, 42), o.random_diagonal_sign(D, 43)
    g = torch.Generator(device="cuda")
    g.manual_seed(5)

    # ---- encode / dequant: 16 793 216 vectors = 2.15e9 elements
    N = (1 << 24) + 16000
    x = torch.randn((N, D), generator=g, device="cuda", dtype=torch.float16)
    packed, norms = tq.fused_quantize(x, dev(vs), b, D, bits)
    deq = tq.dequant_fp16(packed, norms, c, dev(vs), D, bits)
    for lo in (0, N // 2 - 8, N - 64):
        wp, wn = o.fused_quantize(host(x[lo:lo + 64]), vs, b, D, bits)
        assert np.array_equal(host(packed[lo:lo + 64]), wp), lo
        assert np.array_equal(host(norms[lo:lo + 64]), wn), lo
        want = torch.from_numpy(o.packed_dequantize(wp, wn, c, vs, D, bits)).to(torch.float16)
        assert torch.equal(deq[lo:lo + 64].cpu(), want), lo
    del deq

    # ---- V-only decode: fp16 keys of the same 2.15e9 elements (one kv head), a 2000-position sequence at the end
    n_rep, tail = 2, 2000
    offs = torch.tensor([0, N - tail, N], dtype=torch.int32, device="cuda")
    q = torch.randn((2, n_rep, D), generator=g, device="cuda", dtype=torch.float16)
    got = tq.vonly_decode(q, x[None], packed[None], norms[None], c, dev(vs), D, bits, sc, n_rep=n_rep,
                          seq_offsets=offs, max_seq_len=N - tail)
    assert torch.isfinite(got).all()
    want = o.vonly_decode_attention(host(q[1]), host(x[None, N - tail:]), host(packed[None, N - tail:]),
                                    host(norms[None, N - tail:]), c, vs, D, bits, sc)
    close(host(got[1]), want)
    del x, packed, norms

    # ---- flash decode: 165 300 000 packed rows = 2.149e9 words per tensor, a 3000-position sequence at the end
    R, tail = 165_300_000, 3000
    def rand_packed():
        p = torch.randint(0, 1 << 30, (R, 13), generator=g, device="cuda", dtype=torch.int32)
        p[:, 12] &= 0x00FFFFFF                         # the last word holds 8 fields
        return p.view(torch.uint32)
    kp, vp = rand_packed(), rand_packed()
    kn = torch.rand(R, generator=g, device="cuda") * 12 + 6
    vn = torch.rand(R, generator=g, device="cuda") + 0.5
    offs = torch.tensor([0, R - tail, R], dtype=torch.int32, device="cuda")
    qf = torch.randn((2, n_rep, D), generator=g, device="cuda")
    q_rot = tq.prerotate_query(qf.reshape(-1, D), dev(ks)).reshape(2, n_rep, D)
    got = tq.flash_decode(q_rot, kp[None], kn[None], vp[None], vn[None], c, c, dev(vs), D, bits, sc, n_rep=n_rep,
                          seq_offsets=offs, max_seq_len=R - tail)
    assert torch.isfinite(got).all()
    sl = slice(R - tail, R)
    want = o.turboquant_attention_single(host(qf[1]), host(kp[None, sl]), host(kn[None, sl]), host(vp[None, sl]),
                                         host(vn[None, sl]), c, ks, c, vs, D, bits, sc)
    close(host(got[1]), want)


@pytest.mark.parametrize("n_seq,n_kv,n_rep,T,qdt", [(1, 4, 7, 50001, "float16"), (1, 4, 7, 65537, "float32"),
                                                     (2, 2, 4, 98305, "bfloat16"), (1, 8, 1, 26113, "float16")])
def test_vonly_streaming_pass_with_a_ragged_end(tq, n_seq, n_kv, n_rep, T, qdt):
    """Unmasked caches too long for one round of tile workgroups and of a length that is no multiple of the
    streaming pass's range: the last workgroup of a kv head runs through fewer blocks, whole waves (and, at
    T = k * 512 * blocks + 1, whole steps) see no valid row.  Random packed values; against the oracle."""
    rng = np.random.default_rng(T)
    D, bits, sc = 128, 3, 1 / math.sqrt(128)
    c, b = tables(bits)
    vs = o.random_diagonal_sign(D, 43)
    K = rng.standard_normal((n_seq, n_kv, T, D)).astype(np.float16)          # exactly T rows: nothing to read past the end
    vp = o.pack_indices(rng.integers(0, 8, size=(n_seq, n_kv, T, D)).astype(np.uint8), bits)
    vn = ((rng.random((n_seq, n_kv, T)) + 0.5) * np.exp(rng.uniform(-3, 3, size=(n_seq, n_kv, T)))).astype(F32)
    q = torch.from_numpy(rng.standard_normal((n_seq, n_kv * n_rep, D)).astype(F32)).to(getattr(torch, qdt))
    got = host(tq.vonly_decode(q.cuda(), dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc, n_rep=n_rep).float())
    for i in range(n_seq):
        want = o.vonly_decode_attention(q[i].float().numpy(), K[i], vp[i], vn[i], c, vs, D, bits, sc)
        close(got[i], want, rel=(1e-2 if qdt == "bfloat16" else REL), abs_=(4e-3 if qdt == "bfloat16" else ABS), row_scale=True)


@pytest.mark.parametrize("n_seq,n_kv,n_rep,T,qdt", [(4, 8, 2, 10240, "float16"), (3, 8, 1, 18432, "float32")])
def test_vonly_streaming_pass_block_count_that_does_not_divide_the_length(tq, n_seq, n_kv, n_rep, T, qdt):
    """Batches whose length is a multiple of 512 positions but where the block count the divisor rule arrives at leaves
    a short second round of workgroups (20 blocks x 32 pairs in twos: 320 workgroups; 36 x 24 in threes: 288): the host
    then takes the count with the fewest rounds times blocks (three, which does not divide 20: 224 workgroups; four: 216)
    and the any-length form of the streaming pass.  Against the oracle."""
    rng = np.random.default_rng(T + n_seq)
    D, bits, sc = 128, 3, 1 / math.sqrt(128)
    c, b = tables(bits)
    vs = o.random_diagonal_sign(D, 43)
    assert T % 512 == 0
    K = rng.standard_normal((n_seq, n_kv, T, D)).astype(np.float16)
    vp = o.pack_indices(rng.integers(0, 8, size=(n_seq, n_kv, T, D)).astype(np.uint8), bits)
    vn = ((rng.random((n_seq, n_kv, T)) + 0.5) * np.exp(rng.uniform(-3, 3, size=(n_seq, n_kv, T)))).astype(F32)
    q = torch.from_numpy(rng.standard_normal((n_seq, n_kv * n_rep, D)).astype(F32)).to(getattr(torch, qdt))
    got = host(tq.vonly_decode(q.cuda(), dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc, n_rep=n_rep).float())
    for i in range(n_seq):
        want = o.vonly_decode_attention(q[i].float().numpy(), K[i], vp[i], vn[i], c, vs, D, bits, sc)
        close(got[i], want, row_scale=True)


@pytest.mark.parametrize("n_seq,n_kv,n_rep,T,qdt", [(1, 4, 7, 32769, "float16"), (1, 4, 7, 36864, "float32"),
                                                     (1, 4, 7, 40001, "float16"), (1, 4, 7, 49152, "bfloat16"),
                                                     (2, 8, 4, 10241, "float16"), (1, 8, 2, 24576, "float32")])
def test_vonly_wide_workgroups_just_above_a_full_round(tq, n_seq, n_kv, n_rep, T, qdt):
    """Unmasked caches a little too long for one round of 512-position workgroups (more than 256 of them, at most 256
    of 640 or 768 positions) take workgroups of ten or twelve wavefronts: lengths that end inside a workgroup, a
    wavefront, at a tile boundary, and exact multiples; two sequences; against the oracle."""
    rng = np.random.default_rng(T + 7)
    D, bits, sc = 128, 3, 1 / math.sqrt(128)
    c, b = tables(bits)
    vs = o.random_diagonal_sign(D, 43)
    tiles8 = -(-T // 512) * n_kv * n_seq
    assert tiles8 > 256 and -(-T // 768) * n_kv * n_seq <= 256          # the shapes this test is about
    K = rng.standard_normal((n_seq, n_kv, T, D)).astype(np.float16)
    vp = o.pack_indices(rng.integers(0, 8, size=(n_seq, n_kv, T, D)).astype(np.uint8), bits)
    vn = ((rng.random((n_seq, n_kv, T)) + 0.5) * np.exp(rng.uniform(-3, 3, size=(n_seq, n_kv, T)))).astype(F32)
    q = torch.from_numpy(rng.standard_normal((n_seq, n_kv * n_rep, D)).astype(F32)).to(getattr(torch, qdt))
    got = host(tq.vonly_decode(q.cuda(), dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc, n_rep=n_rep).float())
    for i in range(n_seq):
        want = o.vonly_decode_attention(q[i].float().numpy(), K[i], vp[i], vn[i], c, vs, D, bits, sc)
        close(got[i], want, rel=(1e-2 if qdt == "bfloat16" else REL), abs_=(4e-3 if qdt == "bfloat16" else ABS), row_scale=True)
    # the same cache through a longer allocation (cache layout, seq_len < T_alloc): the any-length path with a tail
    if n_seq == 1:
        pad = 300
        Kp = np.concatenate([K, np.zeros((1, n_kv, pad, D), np.float16)], axis=2)
        vpp = np.concatenate([vp, np.zeros((1, n_kv, pad, vp.shape[-1]), vp.dtype)], axis=2)
        vnp = np.concatenate([vn, np.ones((1, n_kv, pad), F32)], axis=2)
        got2 = host(tq.vonly_decode(q.cuda(), dev(Kp), dev(vpp), dev(vnp), c, dev(vs), D, bits, sc, n_rep=n_rep, seq_len=T).float())
        assert np.array_equal(got2, got)


@pytest.mark.parametrize("qdt", ["float16", "float32", "bfloat16"])
@pytest.mark.parametrize("n_kv,n_rep,lens", [
    (4, 7, [4097, 2561, 1025, 7000, 1, 3333, 5121, 6143]),       # every row misalignment; ends inside a step, a wave, a block
    (2, 16, [33000, 511, 512, 513, 20000]),                       # a sequence past 32 768 beside ones around one block
    (8, 1, [9000, 1, 1, 8193])])
def test_vonly_streaming_pass_over_a_ragged_batch(tq, qdt, n_kv, n_rep, lens):
    """An unmasked ragged batch long enough for the streaming pass: sequences start at arbitrary rows (packed rows of
    52 bytes at every multiple of 4 bytes), workgroups past a sequence's end leave at once, the last workgroup of a
    sequence runs through fewer blocks.  Exactly sum(L) rows are stored: nothing may be read past the end.  Each
    sequence against the oracle; and the same batch with an all-zero mask (the single-tile kernels) to the bar."""
    rng = np.random.default_rng(len(lens) * 1000 + n_kv)
    D, bits, sc = 128, 3, 1 / math.sqrt(128)
    lens = np.asarray(lens)
    n_seq = len(lens)
    offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    tot = int(offs[-1])
    c, b = tables(bits)
    vs = o.random_diagonal_sign(D, 43)
    K = rng.standard_normal((n_kv, tot, D)).astype(np.float16)
    vp = o.pack_indices(rng.integers(0, 8, size=(n_kv, tot, D)).astype(np.uint8), bits)
    vn = ((rng.random((n_kv, tot)) + 0.5) * np.exp(rng.uniform(-3, 3, size=(n_kv, tot)))).astype(F32)
    q = torch.from_numpy(rng.standard_normal((n_seq, n_kv * n_rep, D)).astype(F32)).to(getattr(torch, qdt))
    kw = dict(n_rep=n_rep, seq_offsets=dev(offs), max_seq_len=int(lens.max()))
    got = host(tq.vonly_decode(q.cuda(), dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc, **kw).float())
    rel, ab = (1e-2, 4e-3) if qdt == "bfloat16" else (REL, ABS)
    for i in range(n_seq):
        a, e = offs[i], offs[i + 1]
        want = o.vonly_decode_attention(q[i].float().numpy(), K[:, a:e], vp[:, a:e], vn[:, a:e], c, vs, D, bits, sc)
        close(got[i], want, rel=rel, abs_=ab, row_scale=True)
    zero = torch.zeros((n_seq, 1, int(lens.max())), device="cuda")
    tiles = host(tq.vonly_decode(q.cuda(), dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc, mask=zero, **kw).float())
    close(got, tiles, rel=rel, abs_=ab, row_scale=True)


def test_attended_length_beyond_the_tensors_is_refused(tq):
    """The kernels trust seq_len / kv_len: the wrappers refuse a length that the K/V tensors do not hold."""
    rng = np.random.default_rng(12)
    c, ks, vs, K, V, kp, kn, vp, vn = kv_fixture(rng, 2, 100, 128, 3)
    q = dev(rng.standard_normal((1, 2, 128)).astype(np.float16))
    with pytest.raises(ValueError, match="exceeds the 100 rows"):
        tq.vonly_decode(q, dev(K[None]), dev(vp[None]), dev(vn[None]), c, dev(vs), 128, 3, 0.1, seq_len=101)
    with pytest.raises(ValueError, match="exceeds the 100 rows"):
        tq.flash_decode(q.float(), dev(kp[None]), dev(kn[None]), dev(vp[None]), dev(vn[None]), c, c, dev(vs), 128, 3, 0.1,
                        seq_len=4096)
    with pytest.raises(ValueError, match="exceeds the 100 rows"):
        tq.flash_decode_from_q(q, dev(ks), dev(kp[None]), dev(kn[None]), dev(vp[None]), dev(vn[None]), c, c, dev(vs), 128, 3,
                               0.1, seq_len=101)
    with pytest.raises(ValueError, match="exceeds the 100 rows"):
        tq.prefill_attention(dev(rng.standard_normal((2, 4, 128)).astype(np.float16)), dev(kp), dev(kn), dev(vp), dev(vn),
                             c, c, dev(ks), dev(vs), 128, 3, 0.1, n_rep=1, kv_len=101)
    with pytest.raises(ValueError, match="holds 1 sequences"):
        tq.vonly_decode(torch.cat([q, q]), dev(K[None]), dev(vp[None]), dev(vn[None]), c, dev(vs), 128, 3, 0.1)


def test_seq_offsets_are_checked_by_every_ragged_wrapper(tq):
    """An int64 offsets tensor (torch.cumsum's default) would be read as int32 pairs by the kernels: all three ragged
    wrappers refuse it, as they refuse a wrong count; validate_offsets=True also checks order and range."""
    rng = np.random.default_rng(77)
    n_kv, n_rep, D, bits = 2, 2, 128, 3
    lens = [100, 60]
    total = sum(lens)
    c, b = tables(bits)
    ks, vs = o.random_diagonal_sign(D, 42), o.random_diagonal_sign(D, 43)
    X = rng.standard_normal((n_kv * total, D)).astype(np.float16)
    kp, kn = tq.fused_quantize(dev(X), dev(ks), b, D, bits)
    kp, kn = kp.reshape(n_kv, total, -1), kn.reshape(n_kv, total)
    K16 = dev(X.reshape(n_kv, total, D))
    q = dev(rng.standard_normal((2, n_kv * n_rep, D)).astype(np.float32))
    good = torch.tensor([0, 100, 160], dtype=torch.int32, device="cuda")
    calls = {
        "flash_decode": lambda off, **kw: tq.flash_decode(q, kp, kn, kp, kn, c, c, dev(vs), D, bits, 0.1, n_rep=n_rep,
                                                          seq_offsets=off, max_seq_len=100, **kw),
        "flash_decode_from_q": lambda off, **kw: tq.flash_decode_from_q(q, dev(ks), kp, kn, kp, kn, c, c, dev(vs), D, bits, 0.1,
                                                                        n_rep=n_rep, seq_offsets=off, max_seq_len=100, **kw),
        "vonly_decode": lambda off, **kw: tq.vonly_decode(q, K16, kp, kn, c, dev(vs), D, bits, 0.1, n_rep=n_rep,
                                                          seq_offsets=off, max_seq_len=100, **kw),
    }
    for name, call in calls.items():
        ref = call(good, validate_offsets=True)
        assert torch.isfinite(ref).all(), name
        with pytest.raises(ValueError, match="int32"):
            call(torch.cumsum(torch.tensor([0, 100, 60], device="cuda"), 0))             # int64
        with pytest.raises(ValueError, match="n_seq"):
            call(torch.tensor([0, 160], dtype=torch.int32, device="cuda"))
        with pytest.raises(ValueError, match="never decrease"):
            call(torch.tensor([0, 120, 100], dtype=torch.int32, device="cuda"), validate_offsets=True)
        with pytest.raises(ValueError, match="holds"):
            call(torch.tensor([0, 100, 161], dtype=torch.int32, device="cuda"), validate_offsets=True)


@pytest.mark.parametrize("spike_pos", [5, 40, 63, 64 + 33, 300, 511, 700])
@pytest.mark.parametrize("q_dtype", [np.float16, np.float32])
def test_vonly_decode_with_one_dominant_key(tq, spike_pos, q_dtype):
    """One key row equal to 3 q (its score exceeds every other by some 50 log2 units) at positions that fall into
    different waves, score tiles and halves of a wave's run, in full and in ragged tiles: weights travel as fp16
    relative to a per-wave reference, and a reference taken from anything but the true maximum of the run would
    push them out of range here.  Against the oracle, at the 2e-3 / 1e-3 bar."""
    rng = np.random.default_rng(900 + spike_pos)
    n_kv, n_rep, T, D, bits = 2, 4, 777, 128, 3
    c, b = tables(bits)
    vs = o.random_diagonal_sign(D, 43)
    K = rng.standard_normal((n_kv, T, D)).astype(np.float16)
    V = rng.standard_normal((n_kv, T, D)).astype(np.float16)
    q = rng.standard_normal((1, n_kv * n_rep, D)).astype(q_dtype)
    K[0, spike_pos] = (3.0 * q[0, 1]).astype(np.float16)             # head 1 of kv head 0
    K[1, spike_pos] = (3.0 * q[0, n_rep + 2]).astype(np.float16)     # head 2 of kv head 1
    sc = 1 / math.sqrt(D)
    gp, gn = tq.fused_quantize(dev(V.reshape(-1, D)), dev(vs), b, D, bits)
    vp, vn = gp.reshape(n_kv, T, -1), gn.reshape(n_kv, T)
    for L in (T, 512):
        if spike_pos >= L:
            continue
        got = host(tq.vonly_decode(dev(q), dev(K), vp, vn, c, dev(vs), D, bits, sc, n_rep=n_rep, seq_len=L))
        want = o.vonly_decode_attention(q[0], K[:, :L], host(vp)[:, :L], host(vn)[:, :L], c, vs, D, bits, sc)
        assert np.isfinite(got).all()
        close(got[0], want)
