"""GPU parity tests of the matrix-core kernels over PACKED KEYS at widths of 1, 2 and 4 bits (the reference's
caches take bits 1-4 for keys and values alike, cache.py:60, adaptive.py:26): pre-rotated-query scores, the
flash decode step (tile pass, streaming pass, masks, ragged batches, query rotation in the kernel, the
thresholded three-pass form), chunked prefill, and the packed cache's one-call decode step (in-merge insert,
HIP graph replay, empty cache and tile boundary).  Every result is compared with the CPU oracle on the same
seeded inputs: scores to 2e-3 of the score scale (fp16 operands), attention outputs to 2e-3 relative + 1e-3
absolute elementwise, states bit for bit.
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
SC = 1 / math.sqrt(D)
WIDTHS = [1, 2, 4]


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


def rand(shape, seed, dtype=torch.float16):
    rng = np.random.default_rng(seed)
    return torch.from_numpy(rng.standard_normal(shape).astype(F32)).to(dtype).cuda()


def close(got, want, rel=REL, abs_=ABS, extra=0.0):
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    ok = err <= abs_ + rel * np.abs(want) + extra
    assert ok.all(), f"max err {err.max():.3e} (want scale {np.abs(want).max():.3e}), {(~ok).sum()} bad"


def tables(bits):
    c = o.gaussian_codebook(bits)
    return c, o.gaussian_boundaries(c)


def encoded(rng, n_kv, T, bits):
    """Keys and values of N(0,1) data encoded by the oracle at `bits` bits."""
    c, b = tables(bits)
    ks, vs = o.random_diagonal_sign(D, 42), o.random_diagonal_sign(D, 43)
    K = rng.standard_normal((n_kv, T, D)).astype(np.float16)
    V = rng.standard_normal((n_kv, T, D)).astype(np.float16)
    kp, kn = o.fused_quantize(K.reshape(-1, D), ks, b, D, bits)
    vp, vn = o.fused_quantize(V.reshape(-1, D), vs, b, D, bits)
    pd = o.packed_dim(D, bits)
    return c, ks, vs, kp.reshape(n_kv, T, pd), kn.reshape(n_kv, T), vp.reshape(n_kv, T, pd), vn.reshape(n_kv, T)


def random_codes(rng, shape, bits):
    """Packed rows of uniformly drawn levels with norms of the size a cache holds: cheap to make at lengths where
    encoding through the oracle would take minutes."""
    kp = o.pack_indices(rng.integers(0, 1 << bits, size=shape + (D,)).astype(np.uint8), bits)
    vp = o.pack_indices(rng.integers(0, 1 << bits, size=shape + (D,)).astype(np.uint8), bits)
    kn = (rng.random(shape) * 12 + 6).astype(F32)
    vn = (rng.random(shape) + 0.5).astype(F32)
    return kp, kn, vp, vn


def flash_plan(n_seq, n_kv, max_len, ragged, masked=False):
    from tqhip import _lib
    return _lib.load().tq_flash_decode_plan(n_seq, n_kv, max_len, int(ragged), int(masked))


# ------------------------------------------------------------------ scores

@pytest.mark.parametrize("bits", WIDTHS)
@pytest.mark.parametrize("n_kv,n_rep,T", [(4, 7, 2000), (8, 4, 513), (2, 16, 700), (1, 1, 64), (3, 5, 1)])
def test_packed_key_scores_other_widths(tq, bits, n_kv, n_rep, T):
    """prerot_fused_qk_scores (metal_kernels_v4.py:71-113) on the matrix cores: within 2e-3 of the score scale of
    the oracle (operands rounded to half), and the float32 kernel within 1e-5."""
    rng = np.random.default_rng(100 + bits)
    c, ks, vs, kp, kn, vp, vn = encoded(rng, n_kv, T, bits)
    q = rng.standard_normal((n_kv * n_rep, D)).astype(F32)
    q_rot = tq.prerotate_query(dev(q), dev(ks))
    want = o.prerot_fused_qk_scores(o.prerotate_query(q, ks), kp, kn, c, D, bits, n_rep)
    s16 = host(tq.prerot_fused_qk_scores(q_rot, dev(kp), dev(kn), c, D, bits, n_rep=n_rep, precision="fp16"))
    s32 = host(tq.prerot_fused_qk_scores(q_rot, dev(kp), dev(kn), c, D, bits, n_rep=n_rep, precision="fp32"))
    scale = np.abs(want).max()
    assert s16.shape == (n_kv * n_rep, T)
    assert np.abs(s32 - want).max() < 1e-5 * scale
    assert np.abs(s16 - want).max() < 2e-3 * scale


@pytest.mark.parametrize("bits", WIDTHS)
def test_packed_key_scores_other_widths_on_cache_slices(tq, bits):
    """Head strides larger than the valid length (a cache's storage) and a length that ends inside a wave's rows."""
    rng = np.random.default_rng(110 + bits)
    n_kv, n_rep, T, T_alloc = 4, 7, 1000, 1280
    c, ks, vs, kp, kn, vp, vn = encoded(rng, n_kv, T_alloc, bits)
    q = rng.standard_normal((n_kv * n_rep, D)).astype(np.float16)
    q_rot = tq.prerotate_query(dev(q), dev(ks))
    got = host(tq.prerot_fused_qk_scores(q_rot, dev(kp)[:, :T], dev(kn)[:, :T], c, D, bits, n_rep=n_rep))
    want = o.prerot_fused_qk_scores(o.prerotate_query(q, ks), kp[:, :T], kn[:, :T], c, D, bits, n_rep)
    assert np.abs(got - want).max() < 2e-3 * np.abs(want).max()


# ------------------------------------------------------------------ flash decode

@pytest.mark.parametrize("bits", WIDTHS)
@pytest.mark.parametrize("n_kv,n_rep,T,qdt", [(4, 7, 2000, np.float32), (2, 1, 64, np.float32), (1, 16, 513, np.float16),
                                              (8, 4, 1025, np.float32), (2, 3, 1, np.float32)])
def test_flash_decode_other_widths_match_oracle(tq, bits, n_kv, n_rep, T, qdt):
    """flash_attention_turboquant (flash_attention.py:168-274) on the tile pass, and the unfused composition."""
    rng = np.random.default_rng(120 + bits)
    c, ks, vs, kp, kn, vp, vn = encoded(rng, n_kv, T, bits)
    q = rng.standard_normal((n_kv * n_rep, D)).astype(qdt)
    want = o.flash_attention_turboquant(o.prerotate_query(q.astype(F32), ks), kp, kn, vp, vn, c, c, vs, D, bits, SC, 16, n_rep)
    q_rot = tq.prerotate_query(dev(q), dev(ks))
    got = host(tq.flash_attention_turboquant(q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, SC, n_rep=n_rep))
    close(got, want)
    f32 = host(tq.flash_attention_turboquant(q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, SC,
                                             n_rep=n_rep, precision="fp32"))
    close(got, f32)


@pytest.mark.parametrize("bits", WIDTHS)
def test_flash_decode_other_widths_mask_and_cache_layout(tq, bits):
    """Two sequences in cache layout, an additive mask per head with -inf entries, every output dtype."""
    rng = np.random.default_rng(130 + bits)
    n_seq, n_kv, n_rep, T, T_alloc = 2, 4, 7, 1111, 1111 + 13
    n_q = n_kv * n_rep
    parts = [encoded(rng, n_kv, T_alloc, bits) for _ in range(n_seq)]
    c, ks, vs = parts[0][:3]
    kp, kn, vp, vn = [np.stack([p[3 + j] for p in parts]) for j in range(4)]
    mask = np.where(rng.random((n_seq, n_q, T)) < 0.3, -np.inf, 0.0).astype(F32)
    mask[..., 17] = 0.0
    mask = mask + (rng.standard_normal(mask.shape) * 0.5).astype(F32) * np.isfinite(mask)
    q = rng.standard_normal((n_seq, n_q, D)).astype(F32)
    q_rot = tq.prerotate_query(dev(q.reshape(-1, D)), dev(ks)).reshape(n_seq, n_q, D)
    for odt, rel in ((torch.float32, REL), (torch.float16, 3e-3), (torch.bfloat16, 1e-2)):
        got = host(tq.flash_decode(q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, SC, n_rep=n_rep,
                                   seq_len=T, mask=dev(mask), out_dtype=odt))
        for i in range(n_seq):
            want = o.turboquant_attention_single(q[i], kp[i, :, :T], kn[i, :, :T], vp[i, :, :T], vn[i, :, :T], c, ks, c, vs,
                                                 D, bits, SC, mask=mask[i])
            close(got[i], want, rel=rel)


@pytest.mark.parametrize("bits", WIDTHS)
@pytest.mark.parametrize("n_seq,n_kv,n_rep,T", [(2, 8, 2, 16500), (1, 4, 7, 70000)])
def test_flash_streaming_pass_other_widths_cache_layout(tq, bits, n_seq, n_kv, n_rep, T):
    """Lengths at which the host picks the streaming pass; value norms spread over six decades so that the running
    power-of-two scale moves between steps.  The valid length ends inside a step."""
    rng = np.random.default_rng(140 + bits)
    T_alloc = T + 37
    assert flash_plan(n_seq, n_kv, T, False) >= 2
    c, _ = tables(bits)
    ks, vs = o.random_diagonal_sign(D, 42), o.random_diagonal_sign(D, 43)
    kp, kn, vp, vn = random_codes(rng, (n_seq, n_kv, T_alloc), bits)
    vn *= np.exp(rng.uniform(-7, 7, size=vn.shape)).astype(F32)
    q = rng.standard_normal((n_seq, n_kv * n_rep, D)).astype(F32)
    q_rot = tq.prerotate_query(dev(q.reshape(-1, D)), dev(ks)).reshape(n_seq, -1, D)
    got = host(tq.flash_decode(q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, SC, n_rep=n_rep, seq_len=T))
    for i in range(n_seq):
        want = o.turboquant_attention_single(q[i], kp[i, :, :T], kn[i, :, :T], vp[i, :, :T], vn[i, :, :T], c, ks, c, vs,
                                             D, bits, SC)
        err = np.abs(got[i].astype(np.float64) - want)
        assert (err <= ABS + REL * np.abs(want).max(axis=-1, keepdims=True)).all(), err.max()   # rows span decades


@pytest.mark.parametrize("bits", WIDTHS)
def test_flash_streaming_pass_other_widths_ragged_and_misaligned_storage(tq, bits):
    """A ragged batch on the streaming pass: sequences start at arbitrary rows, lengths end inside a step, inside
    a wave's 64 rows and one row past a step.  The same batch from storage that starts 4 bytes off a 16-byte
    boundary (which the host sends to the tile pass at these widths) must give the same result to the bar."""
    rng = np.random.default_rng(150 + bits)
    n_kv, n_rep = 8, 4
    lens = np.array([4097, 2561, 1025, 7000, 1, 3333, 5121, 6143])
    n_seq = len(lens)
    assert flash_plan(n_seq, n_kv, int(lens.max()), True) >= 2
    offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    c, _ = tables(bits)
    ks, vs = o.random_diagonal_sign(D, 42), o.random_diagonal_sign(D, 43)
    kp, kn, vp, vn = random_codes(rng, (n_kv, int(offs[-1])), bits)
    q = rng.standard_normal((n_seq, n_kv * n_rep, D)).astype(F32)
    q_rot = tq.prerotate_query(dev(q.reshape(-1, D)), dev(ks)).reshape(n_seq, n_kv * n_rep, D)
    kw = dict(n_rep=n_rep, seq_offsets=dev(offs), max_seq_len=int(lens.max()))
    got = host(tq.flash_decode(q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, SC, **kw))
    for i in range(n_seq):
        a, e = offs[i], offs[i + 1]
        want = o.flash_attention_turboquant(o.prerotate_query(q[i], ks), kp[:, a:e], kn[:, a:e], vp[:, a:e], vn[:, a:e],
                                            c, c, vs, D, bits, SC, 16, n_rep)
        close(got[i], want)

    def shifted(a):                              # the same words one word further on in a larger buffer
        flat = torch.zeros(a.size + 4, dtype=torch.int32, device="cuda")
        view = flat[1:1 + a.size].view(torch.uint32).reshape(a.shape)
        view.copy_(dev(a))
        assert view.data_ptr() % 16 == 4
        return view
    off = host(tq.flash_decode(q_rot, shifted(kp), dev(kn), shifted(vp), dev(vn), c, c, dev(vs), D, bits, SC, **kw))
    close(off, got)


@pytest.mark.parametrize("bits", WIDTHS)
@pytest.mark.parametrize("n_seq,n_kv,n_rep,T,thr,masked", [(1, 8, 4, 1500, 1e-5, False), (2, 2, 7, 513, 1e-3, True),
                                                           (3, 1, 16, 77, 1e-2, False),
                                                           (4, 8, 2, 9001, 1e-5, False)])   # streaming passes
def test_flash_sparse_decode_other_widths(tq, bits, n_seq, n_kv, n_rep, T, thr, masked):
    """The thresholded decode step over packed keys (scores pass, weights pass, merge pass) against the oracle's
    turboquant_attention with a sparse-V threshold (fused_attention.py:109-121).  A weight within 3e-3 (relative)
    of the threshold may fall on either side of it when the scores come from fp16 operands; such a position may
    move the output by its whole contribution, which is added to the bar."""
    rng = np.random.default_rng(160 + bits)
    n_q = n_kv * n_rep
    parts = [encoded(rng, n_kv, T, bits) for _ in range(n_seq)]
    c, ks, vs = parts[0][:3]
    kp, kn, vp, vn = [np.stack([p[3 + j] for p in parts]) for j in range(4)]
    mask = None
    if masked:
        mask = np.where(rng.random((n_seq, 1, T)) < 0.3, -np.inf, 0.0).astype(F32)
        mask[..., 5] = 0.0
    q = rng.standard_normal((n_seq, n_q, D)).astype(F32)
    q_rot = tq.prerotate_query(dev(q.reshape(-1, D)), dev(ks)).reshape(n_seq, n_q, D)
    got = host(tq.flash_decode(q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, SC, n_rep=n_rep,
                               seq_len=T, mask=None if mask is None else dev(mask), sparse_v_threshold=thr))
    for i in range(n_seq):
        mi = None if mask is None else np.broadcast_to(mask[i], (n_q, T))
        s = o.prerot_fused_qk_scores(o.prerotate_query(q[i], ks), kp[i], kn[i], c, D, bits, n_rep) * F32(SC)
        if mi is not None:
            s = s + mi
        w = o._softmax64(s).astype(F32)
        amb = np.abs(w.astype(np.float64) - thr) <= 3e-3 * thr
        vhat = np.abs(o.packed_dequantize(vp[i].reshape(-1, vp.shape[-1]), vn[i].reshape(-1), c, vs, D, bits)).reshape(n_kv, T, D)
        slack = np.matmul((w * amb).reshape(n_kv, n_rep, T).astype(np.float64), vhat.astype(np.float64)).reshape(-1, D)
        want = o.turboquant_attention_single(q[i], kp[i], kn[i], vp[i], vn[i], c, ks, c, vs, D, bits, SC,
                                             sparse_v_threshold=thr, mask=mi)
        close(got[i], want, extra=slack)


@pytest.mark.parametrize("bits", WIDTHS)
@pytest.mark.parametrize("qdt", ["float32", "float16", "bfloat16"])
@pytest.mark.parametrize("case", ["tile", "stream_ragged", "masked", "threshold"])
def test_flash_decode_from_q_other_widths_equals_prerotate_then_flash(tq, bits, qdt, case):
    """tq_flash_decode_from_q rotates the query inside the attention kernels with the stage order of
    tq_prerotate_query: identical to prerotate_query followed by flash_decode, at every width."""
    rng = np.random.default_rng(sum(map(ord, qdt + case)) + bits)
    n_kv, n_rep = (8, 4) if case == "stream_ragged" else (4, 7)
    n_q = n_kv * n_rep
    c, _ = tables(bits)
    ks, vs = o.random_diagonal_sign(D, 42), o.random_diagonal_sign(D, 43)
    if case == "stream_ragged":
        lens = np.array([4097, 2561, 1025, 7000, 1, 3333, 5121, 6143])
        offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        shape, n_seq = (n_kv, int(offs[-1])), len(lens)
        kw = dict(seq_offsets=dev(offs), max_seq_len=int(lens.max()))
    else:
        n_seq, T = 2, 1111
        shape = (n_seq, n_kv, T + 13)
        kw = dict(seq_len=T)
        if case == "masked":
            m = np.where(rng.random((n_seq, n_q, T)) < 0.3, -np.inf, 0.0).astype(F32)
            m[..., 3] = 0.0
            kw["mask"] = dev(m)
        if case == "threshold":
            kw["sparse_v_threshold"] = 1e-4
    kp, kn, vp, vn = random_codes(rng, shape, bits)
    q = torch.from_numpy(rng.standard_normal((n_seq, n_q, D)).astype(F32)).to(getattr(torch, qdt)).cuda()
    q_rot = tq.prerotate_query(q.reshape(-1, D), dev(ks)).reshape(n_seq, n_q, D)
    two = tq.flash_decode(q_rot, dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, SC, n_rep=n_rep, **kw)
    one = tq.flash_decode_from_q(q, dev(ks), dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(vs), D, bits, SC, n_rep=n_rep, **kw)
    assert torch.equal(one, two)
    assert torch.isfinite(one).all()


# ------------------------------------------------------------------ chunked prefill

@pytest.mark.parametrize("bits", WIDTHS)
@pytest.mark.parametrize("n_kv,n_rep,T,n_rows,pos0", [(2, 2, 300, 300, 0), (2, 4, 1000, 256, 744), (1, 1, 777, 130, 500),
                                                      (2, 2, 2500, 513, 1987)])
def test_prefill_attention_other_widths_match_oracle(tq, bits, n_kv, n_rep, T, n_rows, pos0):
    """Chunked prefill over packed K / V against the oracle's causal attention over the dequantised cache
    (what the reference computes: cache.py:209-218 then stock SDPA)."""
    rng = np.random.default_rng(170 + bits)
    c, ks, vs, kp, kn, vp, vn = encoded(rng, n_kv, T, bits)
    q = rng.standard_normal((n_kv * n_rep, n_rows, D)).astype(np.float16)
    want = o.prefill_attention(q, kp, kn, vp, vn, c, c, ks, vs, D, bits, SC, pos0, n_rep)
    got = tq.prefill_attention(dev(q), dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(ks), dev(vs), D, bits, SC,
                               n_rep=n_rep, q_pos0=pos0, out_dtype=torch.float32)
    assert got.shape == (n_kv * n_rep, n_rows, D)
    close(host(got).reshape(-1, D), want.reshape(-1, D))


@pytest.mark.parametrize("bits", WIDTHS)
def test_prefill_attention_other_widths_noncausal_and_decode_rows(tq, bits):
    """The non-causal form against the oracle, and rows of a causal chunk against single decode steps over their
    prefixes through the float32 flash kernel (an independent code path)."""
    rng = np.random.default_rng(180 + bits)
    n_kv, n_rep, T, n_rows = 2, 2, 640, 64
    c, ks, vs, kp, kn, vp, vn = encoded(rng, n_kv, T, bits)
    q = rng.standard_normal((n_kv * n_rep, n_rows, D)).astype(np.float16)
    args = (dev(kp), dev(kn), dev(vp), dev(vn), c, c, dev(ks), dev(vs), D, bits, SC)
    want = o.prefill_attention(q, kp, kn, vp, vn, c, c, ks, vs, D, bits, SC, T - n_rows, n_rep, causal=False)
    close(host(tq.prefill_attention(dev(q), *args, n_rep=n_rep, causal=False, out_dtype=torch.float32)).reshape(-1, D),
          want.reshape(-1, D))
    got = host(tq.prefill_attention(dev(q), *args, n_rep=n_rep, out_dtype=torch.float32))
    for i in (0, 17, 63):
        L = T - n_rows + i + 1
        q_rot = tq.prerotate_query(dev(q[:, i]), dev(ks))
        ref = host(tq.flash_attention_turboquant(q_rot, dev(kp[:, :L]), dev(kn[:, :L]), dev(vp[:, :L]), dev(vn[:, :L]),
                                                 c, c, dev(vs), D, bits, SC, n_rep=n_rep, precision="fp32"))
        close(got[:, i], ref)


# ------------------------------------------------------------------ the packed cache's one-call decode step

def oracle_step(cache, q1, bits):
    """Attention of the last inserted token's query over the cache's state, per sequence, through the oracle."""
    kp, kn, vp, vn = [t.cpu().numpy() for t in cache.state]
    kq, vq = cache._k_q, cache._v_q
    return [o.turboquant_attention_single(host(q1[s, :, 0]), kp[s].view(np.uint32), kn[s], vp[s].view(np.uint32), vn[s],
                                          np.asarray(kq.centroids.cpu()), kq.signs.cpu().numpy(),
                                          np.asarray(vq.centroids.cpu()), vq.signs.cpu().numpy(), D, bits, SC)
            for s in range(q1.shape[0])]


@pytest.mark.parametrize("bits", WIDTHS)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_packed_cache_decode_step_other_widths(tq, bits, dtype):
    """TurboQuantKVCache.decode_step (tile pass over the old positions + a merge pass that encodes both new rows,
    scores the new key and stores them) against update_and_fetch + turboquant_attention on a twin cache, across a
    growth of the storage: same state bit for bit, output to the bar and against the oracle."""
    B, n_q, n_kv, S0 = 2, 32, 8, 250
    k0, v0 = rand((B, n_kv, S0, D), 800 + bits, dtype), rand((B, n_kv, S0, D), 801 + bits, dtype)
    a, b = tq.TurboQuantKVCache(bits=bits, fused=True), tq.TurboQuantKVCache(bits=bits, fused=True)
    a.update_and_fetch(k0, v0), b.update_and_fetch(k0, v0)
    for i in range(9):                                              # 250 -> 259: grows at 256
        k1, v1, q1 = (rand((B, n_kv, 1, D), 810 + 3 * i, dtype), rand((B, n_kv, 1, D), 811 + 3 * i, dtype),
                      rand((B, n_q, 1, D), 812 + 3 * i, dtype))
        got = a.decode_step(q1, k1, v1, SC)
        b.update_and_fetch(k1, v1)
        want = tq.turboquant_attention(q1, b, SC, fused=True)
        assert got.shape == (B, n_q, 1, D) and got.dtype == dtype
        err = (got.float() - want.float()).abs()
        bar = 1e-3 + (2e-3 if dtype == torch.float16 else 8e-3) * want.float().abs()    # bf16 outputs: one ulp is 2^-8
        assert bool((err <= bar).all()), (i, float(err.max()))
    assert a.offset == b.offset == S0 + 9 and a.v_packed.shape[2] == 512
    assert a.v_packed.shape[-1] == o.packed_dim(D, bits)
    for x, y in zip(a.state, b.state):
        assert torch.equal(x, y)
    for s, ref in enumerate(oracle_step(a, q1, bits)):
        err = np.abs(host(got[s, :, 0]).astype(np.float64) - ref)
        assert (err <= 1e-3 + (2e-3 if dtype == torch.float16 else 6e-3) * np.abs(ref)).all(), err.max()


@pytest.mark.parametrize("bits", WIDTHS)
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_packed_decode_step_other_widths_from_an_empty_cache_and_at_a_tile_boundary(tq, bits, dtype):
    """The in-merge insert from an empty cache (no tile pass) and around the 512-position tile boundary."""
    B, n_q, n_kv = 2, 8, 2
    a, b = tq.TurboQuantKVCache(bits=bits, fused=True), tq.TurboQuantKVCache(bits=bits, fused=True)
    seed = 1300 + 100 * bits
    for grow in (0, 509, 0, 0):                                     # steps at lengths 0, 510, 511, 512
        if grow:
            k0, v0 = rand((B, n_kv, grow, D), seed, dtype), rand((B, n_kv, grow, D), seed + 1, dtype)
            a.update_and_fetch(k0, v0), b.update_and_fetch(k0, v0)
        seed += 5
        k1, v1, q1 = rand((B, n_kv, 1, D), seed + 2, dtype), rand((B, n_kv, 1, D), seed + 3, dtype), rand((B, n_q, 1, D), seed + 4, dtype)
        got = a.decode_step(q1, k1, v1, SC)
        b.update_and_fetch(k1, v1)
        assert a.offset == b.offset
        for x, y in zip(a.state, b.state):
            assert torch.equal(x, y), a.offset
        for s, ref in enumerate(oracle_step(a, q1, bits)):
            err = np.abs(host(got[s, :, 0]).astype(np.float64) - ref)
            assert (err <= 1e-3 + 2e-3 * np.abs(ref)).all(), (a.offset, err.max())
    assert a.offset == 513


@pytest.mark.parametrize("bits", WIDTHS)
@pytest.mark.parametrize("S0,want_alloc", [(300, 1024), (31000, 32768)])
def test_packed_decode_step_other_widths_replayed_from_a_hip_graph(tq, bits, S0, want_alloc):
    """The packed cache's decode step recorded once in a HIP graph with the position in device memory and replayed
    for six tokens, with eager work and synchronisations between the replays: every replay matches the eager step
    on a twin cache, and both caches end in the same state bit for bit.  An insert past the storage is dropped.
    The long case runs the streaming pass, the short one the single-tile pass."""
    B, n_q, n_kv, N = 1, 32, 8, 6
    k0, v0 = rand((B, n_kv, S0, D), 1200 + bits), rand((B, n_kv, S0, D), 1201 + bits)
    cg, ce = tq.TurboQuantKVCache(bits=bits, fused=True), tq.TurboQuantKVCache(bits=bits, fused=True)
    cg.reserve(B, n_kv, want_alloc, D)
    cg.update_and_fetch(k0, v0), ce.update_and_fetch(k0, v0)
    t_alloc = cg.v_packed.shape[2]
    assert t_alloc == want_alloc
    assert (flash_plan(B, n_kv, t_alloc, True) >= 2) == (want_alloc == 32768)
    pos = torch.tensor([S0], dtype=torch.int64, device="cuda")
    qs, ks, vs = rand((B, n_q, 1, D), 1202), rand((B, n_kv, 1, D), 1203), rand((B, n_kv, 1, D), 1204)
    out_s = torch.empty((B, n_q, D), dtype=torch.float16, device="cuda")

    def check(step_no, q, k, v):
        want = ce.decode_step(q, k, v, SC)[:, :, 0].float()
        err = (out_s.float() - want).abs()
        assert bool((err <= 1e-3 + 2e-3 * want.abs()).all()), (step_no, float(err.max()))

    cg.decode_step(qs, ks, vs, SC, position=pos, out=out_s)
    pos.add_(1)
    check(-1, qs, ks, vs)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        cg.decode_step(qs, ks, vs, SC, position=pos, out=out_s)
        pos.add_(1)
    for i in range(N):
        q, k, v = rand((B, n_q, 1, D), 1210 + 3 * i), rand((B, n_kv, 1, D), 1211 + 3 * i), rand((B, n_kv, 1, D), 1212 + 3 * i)
        qs.copy_(q), ks.copy_(k), vs.copy_(v)
        graph.replay()
        check(i, q, k, v)
        torch.cuda.synchronize()
    cg.offset = int(pos.item())
    assert cg.offset == ce.offset == S0 + 1 + N
    for x, y in zip(cg.state, ce.state):
        assert torch.equal(x, y)
    before = [t.clone() for t in (cg.k_packed, cg.k_norms, cg.v_packed, cg.v_norms)]
    pos.fill_(t_alloc)
    graph.replay()
    torch.cuda.synchronize()
    for x, y in zip(before, (cg.k_packed, cg.k_norms, cg.v_packed, cg.v_norms)):
        assert torch.equal(x, y)
    assert bool(torch.isfinite(out_s.float()).all())
