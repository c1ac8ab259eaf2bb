"""GPU parity tests of the V-only decode step at value widths of 1, 2 and 4 bits (the reference takes
bits 1-4, adaptive.py:26, v_only_cache.py:41): the matrix-core tile pass against the CPU oracle and
against the float32 kernels, over every launch shape the host picks from (one tile per workgroup of
four or eight waves, full or ragged; the streaming pass, full or ragged), with masks, ragged batches
and the three query dtypes; the thresholded one-call step and sparse_v_matvec on the matrix cores at
the same widths.  Tolerance: 2e-3 relative + 1e-3 absolute, elementwise, as for 3 bits.  Last, the streaming
encoder and dequantiser at these widths: bit-exact against the oracle and the generic kernels.
"""
import math

import numpy as np
import pytest

torch = pytest.importorskip("torch")

from oracle import polarquant_oracle as o  # noqa: E402

pytestmark = pytest.mark.gpu

F32 = np.float32
REL, ABS = 2e-3, 1e-3
D = 128


@pytest.fixture(scope="module")
def tq():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a GPU: torch.cuda.is_available() is False")
    import tqhip
    return tqhip


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().float().cpu().numpy()


def close(got, want, rel=REL, abs_=ABS):
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    ok = err <= abs_ + rel * np.abs(want)
    assert ok.all(), f"max err {err.max():.3e} (want scale {np.abs(want).max():.3e}), {(~ok).sum()} bad"


def fixture(rng, n_kv, T, bits):
    """fp16 keys, values encoded by the oracle at `bits` bits (norms spread over two decades)."""
    c = o.gaussian_codebook(bits)
    b = o.gaussian_boundaries(c)
    vs = o.random_diagonal_sign(D, 43)
    K = rng.standard_normal((n_kv, T, D)).astype(np.float16)
    V = (rng.standard_normal((n_kv, T, D)) * np.exp(rng.uniform(-2.3, 2.3, size=(n_kv, T, 1)))).astype(np.float16)
    vp, vn = o.fused_quantize(V.reshape(-1, D), vs, b, D, bits)
    pd = o.packed_dim(D, bits)
    return c, vs, K, vp.reshape(n_kv, T, pd), vn.reshape(n_kv, T)


@pytest.mark.parametrize("bits", [1, 2, 4])
@pytest.mark.parametrize("n_kv,n_rep,T,qdt", [(4, 7, 1000, np.float16), (2, 1, 64, np.float16), (1, 9, 257, np.float32),
                                              (8, 4, 513, np.float16), (3, 16, 1, np.float32), (2, 5, 4096, np.float16),
                                              (4, 7, 5000, np.float32)])
def test_vonly_decode_other_widths_match_oracle(tq, bits, n_kv, n_rep, T, qdt):
    rng = np.random.default_rng(300 + bits)
    c, vs, K, vp, vn = fixture(rng, n_kv, T, bits)
    q = rng.standard_normal((1, n_kv * n_rep, D)).astype(qdt)
    sc = 1 / math.sqrt(D)
    got = host(tq.vonly_decode(dev(q), dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc, n_rep=n_rep))
    want = o.vonly_decode_attention(q[0], K, vp, vn, c, vs, D, bits, sc)
    close(got[0], want)
    ref32 = host(tq.vonly_decode(dev(q), dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc, n_rep=n_rep, precision="fp32"))
    close(got[0], ref32[0])


@pytest.mark.parametrize("bits", [1, 2, 4])
def test_vonly_decode_other_widths_bf16_queries_and_output_dtypes(tq, bits):
    rng = np.random.default_rng(310 + bits)
    n_kv, n_rep, T = 4, 7, 777
    c, vs, K, vp, vn = fixture(rng, n_kv, T, bits)
    qt = torch.from_numpy(rng.standard_normal((1, n_kv * n_rep, D)).astype(F32)).to(torch.bfloat16)
    sc = 1 / math.sqrt(D)
    want = o.vonly_decode_attention(qt[0].float().numpy(), K, vp, vn, c, vs, D, bits, sc)
    for od, rel, abs_ in ((torch.float32, REL, ABS), (torch.float16, REL, ABS), (torch.bfloat16, 1e-2, 1e-3)):
        got = host(tq.vonly_decode(qt.cuda(), dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc, n_rep=n_rep, out_dtype=od))
        close(got[0], want, rel, abs_)                     # bf16 outputs carry their own 2^-8 rounding


@pytest.mark.parametrize("bits", [1, 2, 4])
def test_vonly_decode_other_widths_ragged_batch_and_mask(tq, bits):
    rng = np.random.default_rng(320 + bits)
    n_kv, n_rep, n_seq = 4, 7, 4
    sc = 1 / math.sqrt(D)
    lens = rng.integers(10, 900, size=n_seq)
    offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    c, vs, K, vp, vn = fixture(rng, n_kv, int(offs[-1]), bits)
    q = rng.standard_normal((n_seq, n_kv * n_rep, D)).astype(np.float16)
    got = host(tq.vonly_decode(dev(q), dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc, n_rep=n_rep,
                               seq_offsets=dev(offs), max_seq_len=int(lens.max())))
    for i in range(n_seq):
        a, e = offs[i], offs[i + 1]
        close(got[i], o.vonly_decode_attention(q[i], K[:, a:e], vp[:, a:e], vn[:, a:e], c, vs, D, bits, sc))
    # cache layout (B, H, T_alloc, ...) read up to seq_len, with an additive mask per head
    B, T_alloc, total = 2, 1024, 701
    Kb = rng.standard_normal((B, n_kv, T_alloc, D)).astype(np.float16)
    cs, vss, _, vpb, vnb = fixture(rng, B * n_kv, T_alloc, bits)
    vpb, vnb = vpb.reshape(B, n_kv, T_alloc, -1), vnb.reshape(B, n_kv, T_alloc)
    qb = rng.standard_normal((B, n_kv * n_rep, D)).astype(np.float16)
    mask = np.where(rng.random((B, n_kv * n_rep, total)) < 0.3, -np.inf, 0.0).astype(F32)
    mask[..., 5] = 0.0
    got = host(tq.vonly_decode(dev(qb), dev(Kb), dev(vpb), dev(vnb), cs, dev(vss), D, bits, sc, n_rep=n_rep,
                               seq_len=total, mask=dev(mask)))
    for i in range(B):
        close(got[i], o.vonly_decode_attention(qb[i], Kb[i, :, :total], vpb[i, :, :total], vnb[i, :, :total], cs, vss,
                                               D, bits, sc, mask=mask[i]))


@pytest.mark.parametrize("bits", [1, 2, 4])
def test_vonly_streaming_pass_other_widths_over_a_ragged_batch(tq, bits):
    """An unmasked ragged batch long enough for the streaming pass (rows of 16, 32 or 64 bytes: always aligned);
    and from storage 4 bytes off alignment, which goes to the single-tile kernels."""
    rng = np.random.default_rng(330 + bits)
    n_kv, n_rep = 4, 7
    sc = 1 / math.sqrt(D)
    lens = np.array([4097, 2561, 1025, 7000, 1, 3333, 5121, 6143])
    n_seq = len(lens)
    offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    tot = int(offs[-1])
    c = o.gaussian_codebook(bits)
    vs = o.random_diagonal_sign(D, 43)
    K = rng.standard_normal((n_kv, tot, D)).astype(np.float16)
    vp = o.pack_indices(rng.integers(0, 1 << bits, size=(n_kv, tot, D)).astype(np.uint8), bits)
    vn = ((rng.random((n_kv, tot)) + 0.5) * np.exp(rng.uniform(-2, 2, size=(n_kv, tot)))).astype(F32)
    q = rng.standard_normal((n_seq, n_kv * n_rep, D)).astype(np.float16)
    kw = dict(n_rep=n_rep, seq_offsets=dev(offs), max_seq_len=int(lens.max()))
    got = host(tq.vonly_decode(dev(q), dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc, **kw))
    for i in range(n_seq):
        a, e = offs[i], offs[i + 1]
        close(got[i], o.vonly_decode_attention(q[i], K[:, a:e], vp[:, a:e], vn[:, a:e], c, vs, D, bits, sc))
    flat = torch.zeros(vp.size + 4, dtype=torch.int32, device="cuda")
    shifted = flat[1:1 + vp.size].view(torch.uint32).reshape(vp.shape)
    shifted.copy_(dev(vp))
    assert shifted.data_ptr() % 16 == 4
    close(host(tq.vonly_decode(dev(q), dev(K), shifted, dev(vn), c, dev(vs), D, bits, sc, **kw)), got)


@pytest.mark.parametrize("bits", [1, 2, 4])
def test_vonly_decode_other_widths_masked_eight_wave_tiles(tq, bits):
    """20 000 masked positions of 4 kv heads: 160 tiles of 512, the eight-wave shape with the mask reads."""
    rng = np.random.default_rng(325 + bits)
    n_kv, n_rep, T = 4, 7, 20000
    sc = 1 / math.sqrt(D)
    c, vs, K, vp, vn = fixture(rng, n_kv, T, bits)
    q = rng.standard_normal((1, n_kv * n_rep, D)).astype(np.float16)
    mask = np.where(rng.random((1, 1, T)) < 0.3, -np.inf, 0.0).astype(F32)
    mask += (rng.standard_normal((1, 1, T)) * 0.5).astype(F32) * np.isfinite(mask)
    got = host(tq.vonly_decode(dev(q), dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc, n_rep=n_rep, mask=dev(mask)))
    close(got[0], o.vonly_decode_attention(q[0], K, vp, vn, c, vs, D, bits, sc, mask=mask[0]))


# one case per launch shape (28 query / 4 kv heads): eight-wave full tiles, four-wave full tiles, the ragged tile of
# either, the streaming pass over whole blocks and with a ragged end
SHAPES = [(32768, "eight waves, full tiles"), (4096, "four waves, full tiles"), (32769 - 200, "eight waves, ragged end"),
          (40000, "four waves, ragged end"), (65536, "streaming, whole blocks"), (50000, "streaming, ragged end")]


@pytest.mark.parametrize("bits", [1, 2, 4])
@pytest.mark.parametrize("T,shape", SHAPES)
def test_vonly_decode_other_widths_every_launch_shape(tq, bits, T, shape):
    """Values are encoded on the GPU (the generic encoder, bit-exact against the oracle elsewhere) with norms that
    jump by 2^+-6 between 512-position blocks, so the power-of-two norm scale of the streaming pass changes from
    block to block; the oracle sees the same packed words and norms."""
    rng = np.random.default_rng(330 + bits)
    n_kv, n_rep = 4, 7
    c = o.gaussian_codebook(bits)
    b = o.gaussian_boundaries(c)
    vs = o.random_diagonal_sign(D, 43)
    sc = 1 / math.sqrt(D)
    K = rng.standard_normal((n_kv, T, D)).astype(np.float16)
    V = rng.standard_normal((n_kv, T, D)).astype(F32)
    V *= (2.0 ** rng.integers(-6, 7, size=(n_kv, (T + 511) // 512, 1))).repeat(512, axis=1)[:, :T]
    vp, vn = tq.fused_quantize(dev(V.astype(np.float16)).reshape(-1, D), dev(vs), b, D, bits)
    vp, vn = vp.reshape(n_kv, T, -1), vn.reshape(n_kv, T)
    hp, hn = vp.cpu().numpy(), vn.cpu().numpy()
    for qdt in (np.float16, np.float32):
        q = rng.standard_normal((1, n_kv * n_rep, D)).astype(qdt)
        got = host(tq.vonly_decode(dev(q), dev(K), vp, vn, c, dev(vs), D, bits, sc, n_rep=n_rep))
        want = o.vonly_decode_attention(q[0], K, hp, hn, c, vs, D, bits, sc)
        close(got[0], want)


@pytest.mark.parametrize("bits", [2, 4])
def test_vonly_cache_other_widths_decode_through_the_cache(tq, bits):
    """A VOnlyTurboQuantCache of another width: prompt, a few decode steps, attention after each against the oracle
    on the cache's own packed state."""
    rng = np.random.default_rng(340 + bits)
    B, n_kv, n_rep, S = 2, 4, 7, 300
    sc = 1 / math.sqrt(D)
    cache = tq.VOnlyTurboQuantCache(bits=bits, seed=11, no_v_buffer=True)
    k = torch.from_numpy(rng.standard_normal((B, n_kv, S, D)).astype(np.float16)).cuda()
    v = torch.from_numpy(rng.standard_normal((B, n_kv, S, D)).astype(np.float16)).cuda()
    cache.update_and_fetch(k, v)
    for step in range(3):
        k1 = torch.from_numpy(rng.standard_normal((B, n_kv, 1, D)).astype(np.float16)).cuda()
        v1 = torch.from_numpy(rng.standard_normal((B, n_kv, 1, D)).astype(np.float16)).cuda()
        cache.update_and_fetch(k1, v1)
        q = torch.from_numpy(rng.standard_normal((B, n_kv * n_rep, 1, D)).astype(np.float16)).cuda()
        got = host(tq.vonly_decode_attention(q, cache, sc))[:, :, 0, :]
        total = cache.offset
        assert total == S + step + 1
        tqc = cache._v_tq
        keys = cache._k_cache.keys[:, :, :total].cpu().numpy()
        vp, vn = tqc.v_packed[:, :, :total].cpu().numpy(), tqc.v_norms[:, :, :total].cpu().numpy()
        cen, sg = np.asarray(tqc._v_q.centroids, dtype=F32), tqc._v_q.signs.cpu().numpy()
        for bi in range(B):
            want = o.vonly_decode_attention(q[bi, :, 0].cpu().numpy(), keys[bi], vp[bi], vn[bi], cen, sg, D, bits, sc)
            close(got[bi], want)
    # the single-call step (insert + attend): same result as the two halves
    for step in range(2):
        k1 = torch.from_numpy(rng.standard_normal((B, n_kv, 1, D)).astype(np.float16)).cuda()
        v1 = torch.from_numpy(rng.standard_normal((B, n_kv, 1, D)).astype(np.float16)).cuda()
        q = torch.from_numpy(rng.standard_normal((B, n_kv * n_rep, 1, D)).astype(np.float16)).cuda()
        got = host(cache.decode_step(q, k1, v1, sc))[:, :, 0, :]
        total = cache.offset
        assert total == S + 3 + step + 1
        tqc = cache._v_tq
        keys = cache._k_cache.keys[:, :, :total].cpu().numpy()
        vp, vn = tqc.v_packed[:, :, :total].cpu().numpy(), tqc.v_norms[:, :, :total].cpu().numpy()
        assert np.array_equal(keys[:, :, -1], k1[:, :, 0].cpu().numpy())
        for bi in range(B):
            want = o.vonly_decode_attention(q[bi, :, 0].cpu().numpy(), keys[bi], vp[bi], vn[bi], cen, sg, D, bits, sc)
            close(got[bi], want)


# ------------------------------------------------------------------ given weights and the thresholded step

@pytest.mark.parametrize("bits", [1, 2, 4])
@pytest.mark.parametrize("n_seq,n_kv,n_rep,T,thr,qdt", [(1, 4, 7, 1500, 1e-5, np.float16), (2, 2, 4, 513, 1e-3, np.float32),
                                                        (3, 1, 16, 77, 1e-2, np.float16), (1, 4, 7, 4099, 1e-5, np.float32),
                                                        (2, 3, 5, 1, 1e-5, np.float16)])
def test_vonly_thresholded_decode_other_widths_match_oracle(tq, bits, n_seq, n_kv, n_rep, T, thr, qdt):
    """The one-call thresholded step (scores pass, weights-and-values pass, merge; sparse_v.py:59-65 on the final
    weights) at the other widths, cache layout with an allocation longer than the valid length."""
    rng = np.random.default_rng(7 * T + n_rep + bits)
    sc = 1 / math.sqrt(D)
    T_alloc = T + 37
    c, vs, K, vp, vn = fixture(rng, n_seq * n_kv, T_alloc, bits)
    K, vp, vn = (a.reshape(n_seq, n_kv, *a.shape[1:]) for a in (K, vp, vn))
    q = rng.standard_normal((n_seq, n_kv * n_rep, D)).astype(qdt)
    got = host(tq.vonly_decode(dev(q), dev(K), dev(vp), dev(vn), c, dev(vs), D, bits, sc, n_rep=n_rep, seq_len=T,
                               sparse_v_threshold=thr))
    dropped = 0
    for i in range(n_seq):
        want = o.vonly_decode_attention(q[i], K[i, :, :T], vp[i, :, :T], vn[i, :, :T], c, vs, D, bits, sc, threshold=thr)
        dense = o.vonly_decode_attention(q[i], K[i, :, :T], vp[i, :, :T], vn[i, :, :T], c, vs, D, bits, sc)
        dropped += int(np.abs(want - dense).max() > 0)
        close(got[i], want)
    if T >= 500:
        assert dropped > 0                         # the threshold did remove something in these cases


@pytest.mark.parametrize("bits", [1, 2, 4])
def test_sparse_v_matvec_other_widths_on_the_matrix_cores(tq, bits):
    """sparse_v_matvec(precision="fp16") (sparse_v.py:94-186) at the other widths: dense, thresholded, and the
    threshold above every weight; against the oracle and the float32 kernel."""
    rng = np.random.default_rng(350 + bits)
    n_kv, n_rep, T = 4, 7, 3000
    c, vs, K, vp, vn = fixture(rng, n_kv, T, bits)
    x = rng.standard_normal((n_kv * n_rep, T)) * 3
    w = np.exp(x - x.max(-1, keepdims=True))
    w = (w / w.sum(-1, keepdims=True)).astype(F32)
    args = (dev(vp), dev(vn), c, dev(vs), D, bits)
    for thr in (0.0, 1e-4):
        want = o.sparse_v_matvec(w, vp, vn, c, vs, D, bits, thr, n_rep)
        got = host(tq.sparse_v_matvec(dev(w), *args, threshold=thr, n_rep=n_rep, precision="fp16"))
        close(got, want)
        ref = host(tq.sparse_v_matvec(dev(w), *args, threshold=thr, n_rep=n_rep, precision="fp32"))
        assert np.abs(ref - want).max() <= 1e-5 * np.abs(want).max()
    zero = host(tq.sparse_v_matvec(dev(w), *args, threshold=2.0, n_rep=n_rep, precision="fp16"))
    assert (zero == 0).all()


# ------------------------------------------------------------------ streaming encoder / dequantiser at d = 128

def _special_rows(rng, n, b):
    """n x 128 float32 rows: random scales, a zero row, one-hot rows, and 200 rows whose butterfly outputs sit
    within a few ulp of a decision boundary of the given width."""
    x = (rng.standard_normal((n, 128)) * rng.choice([1e-3, 1.0, 300.0], size=(n, 1))).astype(F32)
    x[5] = 0.0
    x[6] = 0.0
    x[6, 127] = -2.5
    x[7] = 0.0
    x[7, 64] = 1e-3
    H = np.array([[1.0 if bin(j & k).count("1") % 2 == 0 else -1.0 for k in range(128)] for j in range(128)])
    for r in range(32, 232):
        z = rng.standard_normal(128)
        z[rng.integers(0, 128)] = float(b[rng.integers(0, len(b))]) * (1 + rng.integers(-3, 4) * 2.0 ** -23) \
            + (rng.integers(-3, 4) * 2.0 ** -24 if len(b) == 1 else 0.0)          # the one-bit boundary is 0
        z *= math.sqrt(128) / np.linalg.norm(z)
        x[r] = (H @ z) / 128.0
    return x


@pytest.mark.parametrize("variant", ["mlx", "metal"])
@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("bits", [1, 2, 4])
def test_streaming_encoder_other_widths_bit_exact(tq, bits, dtype, variant):
    """A row count that is a multiple of 16 takes the streaming encoder at every width (metal.py:14-101 /
    quantizer.py:85-106 for bits 1-4): level = thresholds below a guess cell + one compare, the cell table derived
    from the thresholds on the GPU.  Its words and norms must be the oracle's and those of the generic
    one-wavefront-per-vector kernel (ragged count), special rows included."""
    rng = np.random.default_rng(40 + bits)
    c = o.gaussian_codebook(bits)
    b = o.gaussian_boundaries(c)
    s = o.random_diagonal_sign(128, 43)
    n = 16 * 261
    x = _special_rows(rng, n, b)
    xt = torch.from_numpy(x)
    if dtype == "f16":
        xt = xt.to(torch.float16)
    elif dtype == "bf16":
        xt = xt.to(torch.bfloat16)
    xt[100] = float("nan")
    xt[101, 3] = float("nan")
    if dtype == "f32":
        xt[102] = 3e19                                          # sum of squares overflows float32: the norm is inf
    ref_in = xt.float().numpy()
    ok = ~np.isnan(ref_in).any(axis=1)
    with np.errstate(over="ignore"):
        wp, wn = o.fused_quantize(ref_in[ok], s, b, 128, bits, variant)
    gp, gn = tq.fused_quantize(xt.cuda(), dev(s), b, 128, bits, variant=variant)
    gp, gn = gp.cpu().numpy(), gn.cpu().numpy()
    assert gp.shape == (n, o.packed_dim(128, bits))
    assert np.array_equal(gp[ok], wp) and np.array_equal(gn[ok], wn)
    assert (gp[~ok] == 0).all() and np.isnan(gn[~ok]).all()          # NaN compares false with every threshold
    gp2, gn2 = tq.fused_quantize(xt[: n - 3].cuda(), dev(s), b, 128, bits, variant=variant)
    assert np.array_equal(gp2.cpu().numpy(), gp[: n - 3])
    assert np.array_equal(gn2.cpu().numpy()[ok[: n - 3]], gn[: n - 3][ok[: n - 3]])


@pytest.mark.parametrize("bits", [1, 2, 4])
def test_streaming_encoder_other_widths_every_level_and_custom_tables(tq, bits):
    """Every level of the width is produced on a sweep of one coordinate through the whole range, and a codebook
    whose thresholds admit no guess line (two of them 1e-3 apart) still encodes exactly (generic kernel)."""
    c = o.gaussian_codebook(bits)
    b = o.gaussian_boundaries(c)
    ones = np.ones(128, F32)
    n = 4096
    H = np.array([[1.0 if bin(j & k).count("1") % 2 == 0 else -1.0 for k in range(128)] for j in range(128)])
    rng = np.random.default_rng(60 + bits)
    z = rng.standard_normal((n, 128)) * 0.05
    z[:, 9] = np.linspace(-3.2, 3.2, n)
    x = ((z @ H) / 128.0).astype(F32)
    wp, wn = o.fused_quantize(x, ones, b, 128, bits, "metal")
    gp, gn = tq.fused_quantize(dev(x), dev(ones), b, 128, bits, variant="metal")
    assert np.array_equal(gp.cpu().numpy(), wp) and np.array_equal(gn.cpu().numpy(), wn)
    idx = o.unpack_indices(wp, bits, 128)
    assert set(np.unique(idx[:, 9]).tolist()) == set(range(2 ** bits))
    if bits > 1:
        b2 = np.array(b, dtype=F32).copy()
        b2[1] = b2[0] + 1e-3
        b2 = np.sort(b2)
        wp, wn = o.fused_quantize(x, ones, b2, 128, bits, "metal")
        gp, gn = tq.fused_quantize(dev(x), dev(ones), b2, 128, bits, variant="metal")
        assert np.array_equal(gp.cpu().numpy(), wp) and np.array_equal(gn.cpu().numpy(), wn)


@pytest.mark.parametrize("out", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("bits", [1, 2, 4])
def test_streaming_dequantiser_other_widths_bit_exact(tq, bits, out):
    """packed_dequantize / dequant_fp16 (kernels.py:14-55, metal.py:104-141) at a row count that takes the streaming
    kernel: float32 output equal to the oracle's, 16-bit outputs equal to its rounding, and equal to the generic
    kernel (ragged count)."""
    rng = np.random.default_rng(70 + bits)
    c = o.gaussian_codebook(bits)
    s = o.random_diagonal_sign(128, 43)
    n = 16 * 130
    idx = rng.integers(0, 2 ** bits, size=(n, 128)).astype(np.uint8)
    wp = o.pack_indices(idx, bits)
    wn = (rng.random(n) * 10 + 0.01).astype(F32)
    want = o.packed_dequantize(wp, wn, c, s, 128, bits)
    if out == "f32":
        got = tq.packed_dequantize(dev(wp), dev(wn), c, dev(s), 128, bits)
        assert np.array_equal(got.cpu().numpy(), want)
        rag = tq.packed_dequantize(dev(wp[: n - 5]), dev(wn[: n - 5]), c, dev(s), 128, bits)
        assert np.array_equal(rag.cpu().numpy(), want[: n - 5])
    else:
        td = torch.float16 if out == "f16" else torch.bfloat16
        outbuf = torch.empty((n, 128), dtype=td, device="cuda")
        tq.dequant_into(dev(wp), dev(wn), c, dev(s), outbuf, n_groups=1, rows_per_group=n, packed_group_stride=n,
                        norms_group_stride=n, out_group_stride=n, dim=128, bits=bits)
        assert torch.equal(outbuf.cpu(), torch.from_numpy(want).to(td))


# ------------------------------------------------------------------ the step that inserts its own token

@pytest.mark.parametrize("bits", [1, 2, 4])
def test_vonly_step_with_in_merge_insert_other_widths_hip_graph(tq, bits):
    """decode_step at the other widths is the two-launch form as well (the merge pass encodes and stores the new
    token), with the position in device memory it can be recorded in a HIP graph: every replay matches the float64
    oracle on the cache's own state, and the state is, bit for bit, the one update_and_fetch (the encoder kernels)
    builds from the same tokens."""
    rng = np.random.default_rng(380 + bits)
    B, n_kv, n_rep, S0, N = 2, 4, 7, 300, 6
    n_q = n_kv * n_rep
    sc = 1 / math.sqrt(D)

    def rnd(shape):
        return torch.from_numpy(rng.standard_normal(shape).astype(np.float16)).cuda()
    k0, v0 = rnd((B, n_kv, S0, D)), rnd((B, n_kv, S0, D))
    cg, ce = tq.VOnlyTurboQuantCache(bits=bits, fused=True), tq.VOnlyTurboQuantCache(bits=bits, fused=True)
    cg.reserve(B, n_kv, 1024, D)
    cg.update_and_fetch(k0, v0), ce.update_and_fetch(k0, v0)
    pos = torch.tensor([S0], dtype=torch.int64, device="cuda")
    qs, ks, vs = rnd((B, n_q, 1, D)), rnd((B, n_kv, 1, D)), rnd((B, n_kv, 1, D))
    out_s = torch.empty((B, n_q, D), dtype=torch.float16, device="cuda")

    def check(step_no, q):
        st = ce.state
        vq = ce._v_tq._v_q
        for s_ in range(B):
            ref = o.vonly_decode_attention(q[s_, :, 0].cpu().numpy(), st[0][s_].cpu().numpy(),
                                           st[2][s_].cpu().numpy().view(np.uint32), st[3][s_].cpu().numpy(),
                                           np.asarray(vq.centroids.cpu()), vq.signs.cpu().numpy(), D, bits, sc)
            close(out_s[s_].float().cpu().numpy(), ref)

    cg.decode_step(qs, ks, vs, sc, position=pos, out=out_s)          # eager once: workspace, descriptor
    pos.add_(1)
    ce.update_and_fetch(ks, vs)                                      # the twin goes through the encoder kernels
    check(-1, qs)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        cg.decode_step(qs, ks, vs, sc, position=pos, out=out_s)
        pos.add_(1)
    for i in range(N):
        q, k, v = rnd((B, n_q, 1, D)), rnd((B, n_kv, 1, D)), rnd((B, n_kv, 1, D))
        qs.copy_(q), ks.copy_(k), vs.copy_(v)
        graph.replay()
        ce.update_and_fetch(k, v)
        check(i, q)
        torch.cuda.synchronize()
        assert int(pos.item()) == S0 + 2 + i
    cg.set_offset(S0 + 1 + N)
    assert cg.offset == ce.offset == S0 + 1 + N
    for x, y in zip(cg.state, ce.state):
        assert torch.equal(x, y)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("bits", [1, 2, 4])
def test_vonly_step_other_widths_from_an_empty_cache_and_at_tile_boundaries(tq, bits, dtype):
    """The merge pass that inserts the token, at the other widths: from an empty cache (no tile pass at all), and at
    lengths around the 256- and 512-position tile boundaries, with keys, values and queries of every dtype; the state
    equals the two-call cache's bit for bit and the output matches the float64 oracle."""
    rng = np.random.default_rng(390 + bits)
    B, n_q, n_kv = 2, 8, 2
    sc = 1 / math.sqrt(D)

    def rnd(shape):
        return torch.from_numpy(rng.standard_normal(shape).astype(F32)).to(dtype).cuda()
    a, b = tq.VOnlyTurboQuantCache(bits=bits, fused=True), tq.VOnlyTurboQuantCache(bits=bits, fused=True)
    for grow in (0, 254, 255, 2, 253, 1):                           # steps at lengths 0, 255, 511, 512, 513, 767, 768, 769
        if grow:
            k0, v0 = rnd((B, n_kv, grow, D)), rnd((B, n_kv, grow, D))
            a.update_and_fetch(k0, v0), b.update_and_fetch(k0, v0)
        for _ in range(2 if grow in (2, 1) else 1):
            k1, v1, q1 = rnd((B, n_kv, 1, D)), rnd((B, n_kv, 1, D)), rnd((B, n_q, 1, D))
            got = a.decode_step(q1, k1, v1, sc)
            b.update_and_fetch(k1, v1)
            assert a.offset == b.offset
            st = a.state
            for x, y in zip(st, b.state):
                assert x.dtype == y.dtype and torch.equal(x, y), a.offset
            vq = a._v_tq._v_q
            for s_ in range(B):
                ref = o.vonly_decode_attention(q1[s_, :, 0].float().cpu().numpy(), st[0][s_].cpu().numpy(),
                                               st[2][s_].cpu().numpy().view(np.uint32), st[3][s_].cpu().numpy(),
                                               np.asarray(vq.centroids.cpu()), vq.signs.cpu().numpy(), D, bits, sc)
                close(got[s_, :, 0].float().cpu().numpy(), ref, 8e-3 if dtype == torch.bfloat16 else REL, ABS)
    assert a.offset == 0 + 1 + 254 + 1 + 255 + 1 + 2 + 2 + 253 + 1 + 1 + 2
