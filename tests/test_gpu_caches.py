"""GPU tests of the cache objects and the decode-step compositions, following the reference's
tests/test_core.py:112-181, tests/test_v_only_cache.py and tests/test_fused_attn.py, with the
packed state additionally compared bit-for-bit against the oracle."""
import math

import numpy as np
import pytest

torch = pytest.importorskip("torch")

from oracle import polarquant_oracle as o  # noqa: E402

pytestmark = pytest.mark.gpu
F32 = np.float32


@pytest.fixture(scope="module")
def tq():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a GPU: torch.cuda.is_available() is False")
    import tqhip
    return tqhip


def rand(shape, seed, dtype=torch.float16):
    rng = np.random.default_rng(seed)
    return torch.from_numpy(rng.standard_normal(shape).astype(F32)).to(dtype).cuda()


def host(t):
    return t.detach().float().cpu().numpy()


def cos(a, b):
    a, b = a.astype(np.float64).ravel(), b.astype(np.float64).ravel()
    return float(a @ b / np.linalg.norm(a) / np.linalg.norm(b))


def oracle_pack(x, seed, bits=3, variant="mlx"):
    """x: [B,H,T,D] numpy -> packed [B,H,T,pd], norms [B,H,T] by the oracle."""
    B, H, T, D = x.shape
    c = o.gaussian_codebook(bits)
    p, n = o.fused_quantize(x.reshape(-1, D), o.random_diagonal_sign(D, seed), o.gaussian_boundaries(c), D, bits, variant)
    return p.reshape(B, H, T, -1), n.reshape(B, H, T)


# ------------------------------------------------------------------ TurboQuantKVCache

def test_cache_decode_and_prefill_shapes(tq):
    cache = tq.TurboQuantKVCache(bits=3)
    assert cache.empty() and cache.size() == 0 and cache.state == []
    k, v = rand((1, 4, 8, 128), 0), rand((1, 4, 8, 128), 1)
    ko, vo = cache.update_and_fetch(k, v)                                  # prefill
    assert ko.shape == (1, 4, 8, 128) and vo.shape == (1, 4, 8, 128) and cache.offset == 8
    assert ko.dtype == torch.float16 and not cache.empty()
    assert cache.k_packed.shape == (1, 4, 256, 13) and cache.k_packed.dtype == torch.uint32
    assert cache.k_norms.shape == (1, 4, 256) and cache.k_norms.dtype == torch.float32
    for i in range(5):                                                      # decode
        ko, vo = cache.update_and_fetch(rand((1, 4, 1, 128), 10 + i), rand((1, 4, 1, 128), 20 + i))
    assert cache.offset == 13 and ko.shape == (1, 4, 13, 128)
    assert cos(host(ko[..., :8, :]), host(k)) > 0.7 and cos(host(vo[..., :8, :]), host(v)) > 0.7
    assert cache.compression_ratio > 1.5
    assert abs(cache.compression_ratio - 512 / 112) < 1e-9
    assert cache.nbytes == 1 * 4 * 13 * 56 * 2
    assert cache.is_trimmable() and cache.size() == 13


def test_cache_packed_state_bit_exact_and_incremental_equals_full(tq):
    B, H, D = 2, 4, 128
    k, v = rand((B, H, 300, D), 2), rand((B, H, 300, D), 3)
    cache = tq.TurboQuantKVCache(bits=3, seed=42)
    cache.update_and_fetch(k[..., :290, :], v[..., :290, :])               # grows to 512
    for t in range(290, 300, 2):
        ko, vo = cache.update_and_fetch(k[..., t:t + 2, :], v[..., t:t + 2, :])
    assert cache.offset == 300 and cache.k_packed.shape[2] == 512
    wkp, wkn = oracle_pack(k.cpu().numpy(), 42)
    wvp, wvn = oracle_pack(v.cpu().numpy(), 43)
    st = cache.state
    assert len(st) == 4
    assert np.array_equal(st[0].cpu().numpy(), wkp) and np.array_equal(st[1].cpu().numpy(), wkn)
    assert np.array_equal(st[2].cpu().numpy(), wvp) and np.array_equal(st[3].cpu().numpy(), wvn)
    # incremental buffer == one-shot dequantisation of the same packed data, bit for bit
    c = o.gaussian_codebook(3)
    wk = o.packed_dequantize(wkp.reshape(-1, 13), wkn.reshape(-1), c, o.random_diagonal_sign(D, 42), D, 3)
    assert np.array_equal(ko.cpu().numpy(), wk.reshape(B, H, 300, D).astype(np.float16))
    fresh = tq.TurboQuantKVCache(bits=3, seed=42)
    k2, v2 = fresh.update_and_fetch(k, v)
    assert torch.equal(k2, ko) and torch.equal(v2, vo)


def test_cache_growth_across_step_keeps_old_rows(tq):
    cache = tq.TurboQuantKVCache(bits=3)
    k, v = rand((1, 2, 700, 128), 4), rand((1, 2, 700, 128), 5)
    cache.update_and_fetch(k[..., :250, :], v[..., :250, :])
    cache.update_and_fetch(k[..., 250:260, :], v[..., 250:260, :])          # crosses 256
    cache.update_and_fetch(k[..., 260:700, :], v[..., 260:700, :])          # crosses 512, lands in 768
    assert cache.v_packed.shape[2] == 768
    wvp, wvn = oracle_pack(v.cpu().numpy(), 43)
    assert np.array_equal(cache.state[2].cpu().numpy(), wvp)
    assert np.array_equal(cache.state[3].cpu().numpy(), wvn)


def test_cache_fused_mode_returns_placeholders(tq):
    cache = tq.TurboQuantKVCache(bits=3, fused=True)
    ko, vo = cache.update_and_fetch(rand((1, 4, 16, 128), 6), rand((1, 4, 16, 128), 7))
    assert ko.shape == (1, 4, 16, 128) and float(ko.abs().max()) == 0.0 and float(vo.abs().max()) == 0.0
    assert cache._k_deq_buf is None and cache.k_packed is not None


def test_cache_trim_then_extend(tq):
    cache = tq.TurboQuantKVCache(bits=3)
    k, v = rand((1, 2, 20, 128), 8), rand((1, 2, 20, 128), 9)
    cache.update_and_fetch(k[..., :16, :], v[..., :16, :])
    assert cache.trim(4) == 4 and cache.offset == 12 and cache._v_deq_buf is None
    assert cache.trim(100) == 12 and cache.offset == 0
    cache.update_and_fetch(k[..., :12, :], v[..., :12, :])
    ko, vo = cache.update_and_fetch(k[..., 12:20, :], v[..., 12:20, :])     # S=8 > 4: full dequant path
    wkp, _ = oracle_pack(k.cpu().numpy(), 42)
    assert np.array_equal(cache.state[0].cpu().numpy(), wkp)
    assert ko.shape == (1, 2, 20, 128)


def test_cache_serialisation_roundtrip(tq):
    cache = tq.TurboQuantKVCache(bits=3, seed=7)
    k, v = rand((1, 4, 12, 128), 10), rand((1, 4, 12, 128), 11)
    cache.update_and_fetch(k[..., :8, :], v[..., :8, :])
    assert cache.meta_state == "8,3,7,128,128,float16"
    rest = tq.TurboQuantKVCache.from_state(cache.state, cache.meta_state)
    assert rest.offset == 8 and rest.quant_bits == 3 and rest.seed == 7 and rest.v_only is False
    assert torch.equal(rest.k_packed, cache.state[0])
    ko, vo = rest.update_and_fetch(k[..., 8:12, :], v[..., 8:12, :])        # restored cache extends
    assert rest.offset == 12 and ko.shape == (1, 4, 12, 128)
    wkp, wkn = oracle_pack(k.cpu().numpy(), 7)
    assert np.array_equal(rest.state[0].cpu().numpy(), wkp) and np.array_equal(rest.state[1].cpu().numpy(), wkn)
    with pytest.raises(ValueError, match="Expected 2"):
        tq.TurboQuantKVCache.from_state(cache.state[:3], cache.meta_state)
    bf = tq.TurboQuantKVCache(bits=4)
    bf.update_and_fetch(rand((1, 2, 3, 64), 12, torch.bfloat16), rand((1, 2, 3, 64), 13, torch.bfloat16))
    assert bf.meta_state == "3,4,42,64,64,bfloat16"


def test_cache_masks(tq):
    cache = tq.TurboQuantKVCache(bits=3)
    cache.update_and_fetch(rand((1, 2, 5, 128), 14), rand((1, 2, 5, 128), 15))
    assert cache.make_mask(1) is None and cache.make_mask(4) == "causal"
    m = cache.make_mask(3, return_array=True)
    assert m.shape == (3, 8) and m.dtype == torch.bool
    want = np.array([[j <= 5 + i for j in range(8)] for i in range(3)])
    assert np.array_equal(m.cpu().numpy(), want)
    mw = cache.make_mask(3, window_size=2)
    want_w = np.array([[(j <= 5 + i) and (j > 5 + i - 2) for j in range(8)] for i in range(3)])
    assert np.array_equal(mw.cpu().numpy(), want_w)


def test_cache_from_kvcache(tq):
    kv = tq.KVCache()
    k, v = rand((1, 4, 40, 128), 16), rand((1, 4, 40, 128), 17)
    kv.update_and_fetch(k, v)
    assert kv.keys.shape[2] == 256 and kv.offset == 40
    a = tq.TurboQuantKVCache.from_kvcache(kv, bits=3, seed=42)
    b = tq.TurboQuantKVCache(bits=3, seed=42)
    b.update_and_fetch(k, v)
    assert a.offset == 40 and all(torch.equal(x, y) for x, y in zip(a.state, b.state))
    vo = tq.VOnlyTurboQuantCache.from_kvcache(kv, bits=3)
    assert vo.offset == 40 and torch.equal(vo.state[0], k)
    assert tq.TurboQuantKVCache.from_kvcache(tq.KVCache()).offset == 0


@pytest.mark.parametrize("variant", ["mlx", "metal"])
def test_cache_encode_variant(tq, variant):
    cache = tq.TurboQuantKVCache(bits=3, encode_variant=variant)
    k, v = rand((1, 2, 64, 128), 18), rand((1, 2, 64, 128), 19)
    cache.update_and_fetch(k, v)
    wvp, _ = oracle_pack(v.cpu().numpy(), 43, variant=variant)
    assert np.array_equal(cache.state[2].cpu().numpy(), wvp)


# ------------------------------------------------------------------ VOnlyTurboQuantCache

def test_vonly_cache_roundtrip_and_protocol(tq):
    cache = tq.VOnlyTurboQuantCache(bits=3)
    assert cache.empty()
    k, v = rand((1, 4, 16, 128), 20), rand((1, 4, 16, 128), 21)
    ko, vo = cache.update_and_fetch(k[..., :8, :], v[..., :8, :])
    assert cos(host(ko), host(k[..., :8, :])) > 0.999 and cos(host(vo), host(v[..., :8, :])) > 0.95
    assert torch.equal(ko, k[..., :8, :])
    assert cache.offset == 8 and not cache.empty()
    ko, vo = cache.update_and_fetch(k[..., 8:12, :], v[..., 8:12, :])
    assert cache.offset == 12 and vo.shape == (1, 4, 12, 128)
    assert len(cache.state) == 4 and cache.meta_state.startswith("VOnlyTQ,3,")
    assert cache.meta_state == "VOnlyTQ,3,42,12,3,42,0,128,float16"
    ko, vo = cache.update_and_fetch(k[..., 12:16, :], v[..., 12:16, :])
    assert cache.trim(4) == 4 and cache.offset == 12 and cache.size() == 12
    assert cache.make_mask(1) is None and cache.is_trimmable()
    wvp, wvn = oracle_pack(v.cpu().numpy(), 43)
    assert np.array_equal(cache.state[2].cpu().numpy(), wvp[..., :12, :])
    assert np.array_equal(cache.state[3].cpu().numpy(), wvn[..., :12])


def test_vonly_cache_no_v_buffer(tq):
    a = tq.VOnlyTurboQuantCache(bits=3, no_v_buffer=True)
    b = tq.VOnlyTurboQuantCache(bits=3)
    k, v = rand((1, 4, 12, 128), 22), rand((1, 4, 12, 128), 23)
    for lo, hi in ((0, 8), (8, 9), (9, 12)):
        ka, va = a.update_and_fetch(k[..., lo:hi, :], v[..., lo:hi, :])
        kb, vb = b.update_and_fetch(k[..., lo:hi, :], v[..., lo:hi, :])
    assert a._v_tq._v_deq_buf is None
    assert torch.equal(va, vb) and cos(host(va), host(v)) > 0.95            # test_v_only_cache.py:70-75


def test_vonly_cache_from_state(tq):
    cache = tq.VOnlyTurboQuantCache(bits=3, seed=5)
    k, v = rand((1, 4, 12, 128), 24), rand((1, 4, 12, 128), 25)
    cache.update_and_fetch(k[..., :8, :], v[..., :8, :])
    rest = tq.VOnlyTurboQuantCache.from_state(cache.state, cache.meta_state)
    assert rest.offset == 8 and rest._v_bits == 3 and rest._v_tq.seed == 5
    assert torch.equal(rest._v_tq.v_packed, cache.state[2])                # test_v_only_cache.py:98-118
    ko, vo = rest.update_and_fetch(k[..., 8:12, :], v[..., 8:12, :])
    assert rest.offset == 12 and vo.shape == (1, 4, 12, 128)               # test_v_only_cache.py:120-134
    wvp, _ = oracle_pack(v.cpu().numpy(), 6)
    assert np.array_equal(rest.state[2].cpu().numpy(), wvp)


def test_adaptive_cache_layout(tq):
    caches = tq.make_adaptive_cache(12, bits=3, fp16_layers=2, fused=True)
    kinds = [type(c).__name__ for c in caches]
    assert kinds == ["KVCache"] * 2 + ["TurboQuantKVCache"] * 8 + ["KVCache"] * 2
    assert all(c.fused for c in caches[2:10])

    class Odd:
        def make_cache(self):
            return [object()]
    with pytest.raises(ValueError, match="Incompatible cache type"):
        tq.make_adaptive_cache(4, model=Odd())


# ------------------------------------------------------------------ attention compositions

@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("thr", [None, 1e-5])
def test_turboquant_attention_vs_dense_sdpa(tq, fused, thr):
    """tests/test_fused_attn.py:67-112: attention over the packed cache vs plain SDPA on the
    dequantised K/V, cosine > 0.999; and against the oracle within 2e-3 rel / 1e-3 abs."""
    B, n_q, n_kv, S, D = 2, 8, 4, 512, 128
    sc = 1 / math.sqrt(D)
    k, v = rand((B, n_kv, S, D), 26), rand((B, n_kv, S, D), 27)
    q = rand((B, n_q, 1, D), 28)
    cache = tq.TurboQuantKVCache(bits=3, fused=True)
    cache.update_and_fetch(k, v)
    out = tq.turboquant_attention(q, cache, sc, sparse_v_threshold=thr, fused=fused)
    assert out.shape == (B, n_q, 1, D) and out.dtype == q.dtype
    plain = tq.TurboQuantKVCache(bits=3)
    kd, vd = plain.update_and_fetch(k, v)
    ref = o.dense_attention(host(q)[0], host(kd)[0], host(vd)[0], sc)
    assert cos(host(out)[0], ref) > 0.999
    kp, kn, vp, vn = [t.cpu().numpy() for t in cache.state]
    c = o.gaussian_codebook(3)
    for b in range(B):
        want = o.turboquant_attention_single(host(q)[b, :, 0], kp[b], kn[b], vp[b], vn[b], c,
                                             o.random_diagonal_sign(D, 42), c, o.random_diagonal_sign(D, 43),
                                             D, 3, sc, sparse_v_threshold=thr)
        err = np.abs(host(out)[b, :, 0] - want)
        assert (err <= 1e-3 + 2e-3 * np.abs(want)).all()


def test_turboquant_attention_masks_and_v_buffer(tq):
    B, n_q, n_kv, S, D = 2, 4, 2, 200, 128
    sc = 1 / math.sqrt(D)
    k, v = rand((B, n_kv, S, D), 29), rand((B, n_kv, S, D), 30)
    q = rand((B, n_q, 1, D), 31, torch.float32)
    cache = tq.TurboQuantKVCache(bits=3, fused=True)
    cache.update_and_fetch(k, v)
    rng = np.random.default_rng(0)
    m4 = torch.from_numpy(np.where(rng.random((B, 1, 1, S)) < 0.3, -np.inf, 0).astype(F32)).cuda()
    a = tq.turboquant_attention(q, cache, sc, mask=m4)
    b = tq.turboquant_attention(q, cache, sc, mask=m4, fused=True)      # fp16 matrix-core kernel
    assert (np.abs(host(a) - host(b)) <= 1e-3 + 2e-3 * np.abs(host(a))).all()
    kp, kn, vp, vn = [t.cpu().numpy() for t in cache.state]
    c = o.gaussian_codebook(3)
    for i in range(B):
        want = o.turboquant_attention_single(host(q)[i, :, 0], kp[i], kn[i], vp[i], vn[i], c,
                                             o.random_diagonal_sign(D, 42), c, o.random_diagonal_sign(D, 43),
                                             D, 3, sc, mask=host(m4)[i, 0])
        assert np.abs(host(a)[i, :, 0] - want).max() < 1e-4
    m3 = m4[:, 0]                                                            # (B, 1, S)
    assert np.abs(host(tq.turboquant_attention(q, cache, sc, mask=m3)) - host(a)).max() < 1e-6
    plain = tq.TurboQuantKVCache(bits=3)
    kd, vd = plain.update_and_fetch(k, v)
    vb = tq.turboquant_attention(q, cache, sc, v_buffer=vd.float())
    nb = tq.turboquant_attention(q, cache, sc)
    assert np.abs(host(vb) - host(nb)).max() < 5e-3


@pytest.mark.parametrize("thr", [None, 1e-5])
def test_vonly_decode_attention_on_cache(tq, thr):
    B, n_q, n_kv, S, D = 2, 28, 4, 1500, 128
    sc = 1 / math.sqrt(D)
    k, v = rand((B, n_kv, S, D), 32), rand((B, n_kv, S, D), 33)
    q = rand((B, n_q, 1, D), 34)
    cache = tq.VOnlyTurboQuantCache(bits=3)
    cache.update_and_fetch(k[..., :1498, :], v[..., :1498, :])
    cache.update_and_fetch(k[..., 1498:, :], v[..., 1498:, :])
    out = tq.vonly_decode_attention(q, cache, sc, sparse_v_threshold=thr)
    assert out.shape == (B, n_q, 1, D) and out.dtype == torch.float16
    st = cache.state
    c = o.gaussian_codebook(3)
    for b in range(B):
        want = o.vonly_decode_attention(host(q)[b, :, 0], host(st[0])[b], st[2].cpu().numpy()[b],
                                        st[3].cpu().numpy()[b], c, o.random_diagonal_sign(D, 43), D, 3, sc,
                                        threshold=thr or 0.0)
        err = np.abs(host(out)[b, :, 0] - want)
        assert (err <= 1e-3 + 2e-3 * np.abs(want)).all()
    # against attention on the cache's own (fp16 K, dequantised V) outputs: cosine > 0.999
    ko, vo = cache._k_cache.keys[..., :S, :], cache._v_tq._v_deq_buf[..., :S, :]
    ref = o.dense_attention(host(q)[0], host(ko)[0], host(vo)[0], sc)
    assert cos(host(out)[0], ref) > 0.999


# ------------------------------------------------------------------ prefill off the packed cache, dispatcher

def test_prefill_attention_on_cache_two_chunks(tq):
    """A prompt fed in two chunks through a fused cache: each chunk's attention comes from the packed
    storage and must equal the oracle's dense attention over the dequantised cache with the offset
    causal mask (what the reference's non-fused prefill computes, cache.py:209-218 + SDPA)."""
    B, n_q, n_kv, D = 2, 8, 4, 128
    sc = 1 / math.sqrt(D)
    chunks = (320, 200)
    cache = tq.TurboQuantKVCache(bits=3, fused=True)
    c = o.gaussian_codebook(3)
    ks, vs = o.random_diagonal_sign(D, 42), o.random_diagonal_sign(D, 43)
    seed = 60
    for S in chunks:
        k, v, q = rand((B, n_kv, S, D), seed), rand((B, n_kv, S, D), seed + 1), rand((B, n_q, S, D), seed + 2)
        seed += 3
        cache.update_and_fetch(k, v)
        out = tq.turboquant_prefill_attention(q, cache, sc)
        assert out.shape == (B, n_q, S, D) and out.dtype == q.dtype
        kp, kn, vp, vn = [t.cpu().numpy() for t in cache.state]
        for b in range(B):
            want = o.prefill_attention(host(q)[b], kp[b], kn[b], vp[b], vn[b], c, c, ks, vs, D, 3, sc,
                                       cache.offset - S, n_q // n_kv)
            err = np.abs(host(out)[b] - want)
            scale = np.abs(want).max(axis=-1, keepdims=True)
            assert (err <= 1e-3 + 3e-3 * scale).all(), (err / scale).max()      # fp16 output rounding included


def test_sdpa_dispatcher_routes_by_cache(tq):
    """patch.py:14-41: the dispatcher sends a fused cache's decode step to turboquant_attention, its
    multi-token step to the packed prefill, a V-only cache's decode step to the fused V-only kernel,
    and everything else to stock SDPA; apply_patch / remove_patch install and restore it."""
    import types
    from tqhip import patch
    B, n_q, n_kv, S, D = 1, 8, 4, 256, 128
    sc = 1 / math.sqrt(D)
    k, v = rand((B, n_kv, S, D), 70), rand((B, n_kv, S, D), 71)
    qs, q1 = rand((B, n_q, S, D), 72), rand((B, n_q, 1, D), 73)
    k1, v1 = rand((B, n_kv, 1, D), 74), rand((B, n_kv, 1, D), 75)

    fused = tq.TurboQuantKVCache(bits=3, fused=True)
    kk, vv = fused.update_and_fetch(k, v)
    out = patch.scaled_dot_product_attention(qs, kk, vv, fused, sc, fused.make_mask(S))
    assert torch.equal(out, tq.turboquant_prefill_attention(qs, fused, sc))
    kk, vv = fused.update_and_fetch(k1, v1)
    out = patch.scaled_dot_product_attention(q1, kk, vv, fused, sc, fused.make_mask(1))
    assert torch.equal(out, tq.turboquant_attention(q1, fused, sc, fused=True))
    with pytest.raises(ValueError):
        patch.scaled_dot_product_attention(qs, kk, vv, fused, sc, torch.ones((S, S + 1), dtype=torch.bool, device="cuda"))

    plain = tq.TurboQuantKVCache(bits=3)
    kd, vd = plain.update_and_fetch(k, v)
    out = patch.scaled_dot_product_attention(qs, kd, vd, plain, sc, plain.make_mask(S))
    ref = o.dense_attention(host(qs)[0], host(kd)[0], host(vd)[0], sc,
                            np.where(np.tril(np.ones((S, S))) > 0, 0.0, -np.inf))
    assert np.abs(host(out)[0] - ref).max() < 5e-3
    # the packed prefill and stock SDPA over the dequantised cache agree (same quantised K/V)
    assert cos(host(tq.turboquant_prefill_attention(qs, fused_like(tq, k, v), sc))[0], ref) > 0.9995

    vo = tq.VOnlyTurboQuantCache(bits=3)
    vo.update_and_fetch(k, v)
    kk, vv = vo.update_and_fetch(k1, v1)
    out = patch.scaled_dot_product_attention(q1, kk, vv, vo, sc, None)
    assert torch.equal(out, tq.vonly_decode_attention(q1, vo, sc))

    mod = types.SimpleNamespace(scaled_dot_product_attention="original")
    bare = types.SimpleNamespace()
    tq.apply_patch(mod, bare)
    tq.apply_patch(mod)                                    # idempotent
    assert mod.scaled_dot_product_attention is patch.scaled_dot_product_attention
    assert bare.scaled_dot_product_attention is patch.scaled_dot_product_attention
    tq.remove_patch()
    assert mod.scaled_dot_product_attention == "original" and not hasattr(bare, "scaled_dot_product_attention")


def fused_like(tq, k, v):
    cache = tq.TurboQuantKVCache(bits=3, fused=True)
    cache.update_and_fetch(k, v)
    return cache


def test_vonly_cache_fused_mode(tq):
    """fused=True on a V-only cache: values are only encoded (placeholder returned), the packed state
    is the unfused cache's, decode attention is identical, and a multi-token step through the
    dispatcher dequantises on demand."""
    from tqhip import patch
    B, n_q, n_kv, S, D = 1, 8, 4, 300, 128
    sc = 1 / math.sqrt(D)
    k, v = rand((B, n_kv, S, D), 80), rand((B, n_kv, S, D), 81)
    k1, v1 = rand((B, n_kv, 1, D), 82), rand((B, n_kv, 1, D), 83)
    q1, qs = rand((B, n_q, 1, D), 84), rand((B, n_q, S, D), 85)
    plain, fused = tq.VOnlyTurboQuantCache(bits=3), tq.VOnlyTurboQuantCache(bits=3, fused=True)
    kp_, vp_ = plain.update_and_fetch(k, v)
    kf_, vf_ = fused.update_and_fetch(k, v)
    assert torch.equal(kp_, kf_) and vf_.shape == vp_.shape and float(vf_.abs().max()) == 0.0
    assert vf_.untyped_storage().nbytes() == vf_.element_size()          # one element, expanded
    assert torch.equal(fused.dequantized_values(torch.float16), vp_)
    # multi-token step: stock SDPA over K and the on-demand dequantised V
    a = patch.scaled_dot_product_attention(qs, kf_, vf_, fused, sc, "causal")
    b = patch.scaled_dot_product_attention(qs, kp_, vp_, plain, sc, "causal")
    assert torch.equal(a, b)
    plain.update_and_fetch(k1, v1)
    kf_, vf_ = fused.update_and_fetch(k1, v1)
    assert fused.offset == S + 1 and vf_.shape == (B, n_kv, S + 1, D)
    for x, y in zip(plain.state, fused.state):
        assert torch.equal(x, y)
    assert torch.equal(tq.vonly_decode_attention(q1, fused, sc), tq.vonly_decode_attention(q1, plain, sc))
    assert torch.equal(patch.scaled_dot_product_attention(q1, kf_, vf_, fused, sc, None),
                       tq.vonly_decode_attention(q1, plain, sc))


def test_vonly_cache_with_a_bf16_model(tq):
    """bf16 keys, values and queries: keys are stored as float16 (exactly), values are dequantised in bf16,
    a decode step runs on the matrix-core path and matches the oracle on the bf16 inputs, and a multi-token
    step through the dispatcher works on mixed dtypes."""
    from tqhip import patch
    B, n_q, n_kv, S, D = 1, 8, 4, 600, 128
    sc = 1 / math.sqrt(D)
    bf = lambda shape, seed: rand(shape, seed).to(torch.bfloat16)
    k, v, q1, qs = bf((B, n_kv, S, D), 90), bf((B, n_kv, S, D), 91), bf((B, n_q, 1, D), 92), bf((B, n_q, 16, D), 93)
    cache = tq.VOnlyTurboQuantCache(bits=3, fused=True)
    k_out, v_out = cache.update_and_fetch(k, v)
    assert k_out.dtype == torch.float16 and torch.equal(k_out.float(), k.float())       # bf16 -> fp16 is exact here
    assert v_out.dtype == torch.bfloat16
    got = patch.scaled_dot_product_attention(q1, k_out, v_out, cache, sc, None)
    assert got.dtype == torch.bfloat16 and got.shape == (B, n_q, 1, D)
    vq = cache._v_tq._v_q
    want = o.vonly_decode_attention(q1[0, :, 0].float().cpu().numpy(), k[0].float().cpu().numpy().astype(np.float16),
                                    cache._v_tq.v_packed[0, :, :S].cpu().numpy().view(np.uint32),
                                    cache._v_tq.v_norms[0, :, :S].cpu().numpy(), np.asarray(vq.centroids.cpu()),
                                    vq.signs.cpu().numpy(), D, 3, sc)
    err = np.abs(got[0, :, 0].float().cpu().numpy().astype(np.float64) - want)
    assert (err <= 1e-3 + 6e-3 * np.abs(want)).all(), err.max()
    multi = patch.scaled_dot_product_attention(qs, k_out, v_out, cache, sc, None)
    assert multi.dtype == torch.bfloat16 and multi.shape == (B, n_q, 16, D) and bool(torch.isfinite(multi.float()).all())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_packed_cache_with_bf16_and_float32_models(tq, dtype):
    """A fused TurboQuantKVCache under a bf16 / float32 model: the prompt chunk and a decode step through the
    dispatcher return the model's dtype and agree with stock SDPA over the dequantised cache of an unfused
    twin (same packed state)."""
    from tqhip import patch
    B, n_q, n_kv, S, D = 1, 8, 4, 200, 128
    sc = 1 / math.sqrt(D)
    mk = lambda shape, seed: rand(shape, seed).to(dtype)
    k, v, qs = mk((B, n_kv, S, D), 95), mk((B, n_kv, S, D), 96), mk((B, n_q, S, D), 97)
    k1, v1, q1 = mk((B, n_kv, 1, D), 98), mk((B, n_kv, 1, D), 99), mk((B, n_q, 1, D), 100)
    fused, plain = tq.TurboQuantKVCache(bits=3, fused=True), tq.TurboQuantKVCache(bits=3)
    kk, vv = fused.update_and_fetch(k, v)
    kd, vd = plain.update_and_fetch(k, v)
    assert torch.equal(fused.k_packed.view(torch.int32), plain.k_packed.view(torch.int32))
    a = patch.scaled_dot_product_attention(qs, kk, vv, fused, sc, "causal")
    b = patch.scaled_dot_product_attention(qs, kd, vd, plain, sc, "causal")
    assert a.dtype == dtype and b.dtype == dtype
    assert cos(host(a), host(b)) > 0.9995
    kk, vv = fused.update_and_fetch(k1, v1)
    kd, vd = plain.update_and_fetch(k1, v1)
    a = patch.scaled_dot_product_attention(q1, kk, vv, fused, sc, None)
    b = patch.scaled_dot_product_attention(q1, kd, vd, plain, sc, None)
    assert a.dtype == dtype and a.shape == (B, n_q, 1, D)
    assert cos(host(a), host(b)) > 0.9995


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_vonly_cache_single_launch_append(tq, dtype):
    """Decode-sized inserts of a fused V-only cache go through tq_vonly_append (one launch): across a
    growth boundary and for 1, 3 and 16 tokens per step the stored keys, raw values, packed words and
    norms equal those of the unfused cache (slice assignments + encoder) bit for bit, and the packed
    words and norms equal the oracle's."""
    B, n_kv, D = 2, 4, 128
    plain, fused = tq.VOnlyTurboQuantCache(bits=3), tq.VOnlyTurboQuantCache(bits=3, fused=True)
    ks, vs = [], []
    for i, S in enumerate([250, 1, 3, 1, 1, 16, 1, 5]):             # 250 -> 278: grows at 256
        k, v = rand((B, n_kv, S, D), 500 + 2 * i, dtype), rand((B, n_kv, S, D), 501 + 2 * i, dtype)
        ks.append(k), vs.append(v)
        plain.update_and_fetch(k, v)
        k_out, v_out = fused.update_and_fetch(k, v)
        assert fused.offset == plain.offset and k_out.shape[2] == fused.offset and v_out.shape[2] == fused.offset
    assert fused._k_cache.keys.shape[2] == 512 and fused._v_tq.v_packed.shape[2] == 512
    for x, y in zip(plain.state, fused.state):
        assert x.dtype == y.dtype and torch.equal(x, y)
    v_all = torch.cat(vs, dim=2)
    want_p, want_n = oracle_pack(host(v_all), 43)
    st = fused.state
    assert np.array_equal(st[2].cpu().numpy().view(np.uint32), want_p)
    assert np.array_equal(st[3].cpu().numpy(), want_n)
    assert torch.equal(st[0], torch.cat(ks, dim=2).to(torch.float16))
    assert torch.equal(st[1], v_all)


def test_vonly_append_c_abi_other_shapes(tq):
    """tq_vonly_append through ops.vonly_append_into at d = 64 / 2-bit and d = 256 / 4-bit, without the
    raw value copy, at a position inside the storage: rows outside the inserted range stay untouched."""
    from tqhip import ops
    for D, bits, seed in ((64, 2, 7), (256, 4, 8)):
        B, H, T, S, pos = 1, 3, 40, 5, 17
        pd = ops.packed_dim(D, bits)
        k, v = rand((B, H, S, D), 600 + D), rand((B, H, S, D), 601 + D, torch.float32)
        signs = torch.from_numpy(o.random_diagonal_sign(D, seed)).cuda()
        c = o.gaussian_codebook(bits)
        bnd = o.gaussian_boundaries(c)
        k16 = torch.full((B, H, T, D), 7.0, dtype=torch.float16, device="cuda")
        vp = torch.full((B, H, T, pd), 123, dtype=torch.int32, device="cuda").view(torch.uint32)
        vn = torch.full((B, H, T), -1.0, dtype=torch.float32, device="cuda")
        ops.vonly_append_into(k, v, signs, bnd, k16, None, vp, vn, position=pos, bits=bits)
        want_p, want_n = o.fused_quantize(host(v).reshape(-1, D), o.random_diagonal_sign(D, seed), bnd, D, bits, "mlx")
        got_p = vp.cpu().numpy().view(np.uint32)
        assert np.array_equal(got_p[:, :, pos:pos + S], want_p.reshape(B, H, S, pd))
        assert np.array_equal(vn.cpu().numpy()[:, :, pos:pos + S], want_n.reshape(B, H, S))
        assert torch.equal(k16[:, :, pos:pos + S], k)
        keep = np.ones(T, bool); keep[pos:pos + S] = False
        assert (got_p[:, :, keep] == 123).all() and (vn.cpu().numpy()[:, :, keep] == -1.0).all()
        assert bool((k16[:, :, torch.from_numpy(keep).cuda()] == 7.0).all())
    with pytest.raises(ValueError):
        ops.vonly_append_into(k, v, signs, bnd, k16, None, vp, vn, position=T - 2, bits=bits)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_vonly_cache_decode_step_is_update_plus_attention(tq, dtype):
    """decode_step (tq_vonly_decode_step: the tile pass over the old positions + a merge pass that encodes,
    stores and attends the new token itself) agrees, step after step and across a growth of the storage, with
    update_and_fetch + vonly_decode_attention on a twin cache to the 2e-3 / 1e-3 bar (the new token's score is
    taken in float32 there, on the matrix cores here), leaves the very same state behind, and its output
    matches the float64 oracle."""
    B, n_q, n_kv, D, S0 = 2, 28, 4, 128, 250
    sc = 1 / math.sqrt(D)
    k0, v0 = rand((B, n_kv, S0, D), 700, dtype), rand((B, n_kv, S0, D), 701, dtype)
    a, b = tq.VOnlyTurboQuantCache(bits=3, fused=True), tq.VOnlyTurboQuantCache(bits=3, fused=True)
    a.update_and_fetch(k0, v0), b.update_and_fetch(k0, v0)
    for i in range(9):                                              # 250 -> 259: grows at 256
        k1, v1, q1 = rand((B, n_kv, 1, D), 710 + 3 * i, dtype), rand((B, n_kv, 1, D), 711 + 3 * i, dtype), rand((B, n_q, 1, D), 712 + 3 * i, dtype)
        got = a.decode_step(q1, k1, v1, sc)
        b.update_and_fetch(k1, v1)
        want = tq.vonly_decode_attention(q1, b, sc)
        assert got.shape == (B, n_q, 1, D) and got.dtype == dtype
        err = (got.float() - want.float()).abs()
        bar = 1e-3 + (2e-3 if dtype == torch.float16 else 8e-3) * want.float().abs()    # bf16 outputs: one ulp is 2^-8
        assert bool((err <= bar).all()), (i, float(err.max()))
    assert a.offset == b.offset == S0 + 9 and a._k_cache.keys.shape[2] == 512
    for x, y in zip(a.state, b.state):
        assert torch.equal(x, y)
    st = a.state
    vq = a._v_tq._v_q
    for s in range(B):
        ref = o.vonly_decode_attention(host(q1[s, :, 0]), st[0][s].cpu().numpy(), st[2][s].cpu().numpy().view(np.uint32),
                                       st[3][s].cpu().numpy(), np.asarray(vq.centroids.cpu()), vq.signs.cpu().numpy(), D, 3, sc)
        err = np.abs(host(got[s, :, 0]).astype(np.float64) - ref)
        tol = 1e-3 + (2e-3 if dtype == torch.float16 else 6e-3) * np.abs(ref)
        assert (err <= tol).all(), err.max()
    # a step that the single call does not cover (two new tokens) falls back to the two calls
    with pytest.raises(ValueError):
        a.decode_step(rand((B, n_q, 2, D), 1), rand((B, n_kv, 2, D), 2, dtype), rand((B, n_kv, 2, D), 3, dtype), sc)


def test_vonly_decode_step_refuses_bad_positions(tq):
    from tqhip import ops
    B, H, T, D = 1, 2, 256, 128
    sg = o.random_diagonal_sign(D, 43)
    signs = torch.from_numpy(sg).cuda()
    c = o.gaussian_codebook(3)
    bnd = o.gaussian_boundaries(c)
    step = ops.VOnlyStep(torch.zeros((B, H, T, D), dtype=torch.float16, device="cuda"), None,
                         torch.zeros((B, H, T, 13), dtype=torch.int32, device="cuda").view(torch.uint32),
                         torch.zeros((B, H, T), device="cuda"), signs, bnd, c, n_rep=2, bits=3)
    k, v, qq = rand((B, H, D), 1), rand((B, H, D), 2), rand((B, 4, D), 3)
    with pytest.raises(ValueError):
        ops.vonly_decode_step(step, k, v, qq, T, 0.1)
    with pytest.raises(ValueError):
        ops.vonly_decode_step(step, k, v, rand((B, 5, D), 3), 0, 0.1)
    out = ops.vonly_decode_step(step, k, v, qq, 0, 0.1)             # one position: weight 1 -> out = dequant(v)
    p, n = o.fused_quantize(host(v).reshape(-1, D), sg, bnd, D, 3, "mlx")
    want = o.packed_dequantize(p, n, c, sg, D, 3)
    assert out.shape == (B, 4, D)
    for h in range(4):
        assert np.allclose(host(out[0, h]), want[h // 2], rtol=2e-3, atol=1e-3)


def _offset_view(t, n_elems=1):
    """The same values in a contiguous tensor whose storage starts n_elems elements past a fresh allocation:
    4 bytes off a 16-byte boundary for float32, 2 bytes for fp16."""
    buf = torch.empty(t.numel() + n_elems, dtype=t.dtype, device=t.device)
    view = buf[n_elems:].view(t.shape)
    view.copy_(t)
    assert view.is_contiguous() and view.data_ptr() % 16 == n_elems * t.element_size()
    return view


@pytest.mark.parametrize("qdt", [torch.float32, torch.float16])
def test_vonly_entries_with_a_query_off_the_16_byte_boundary(tq, qdt):
    """The matrix-core V-only kernels read q in 16-byte pieces.  A q view one element past a boundary must never
    reach them: tq_vonly_decode_attn and tq_vonly_decode_step serve it through the float32 kernels (same result
    to the bar), tq_vonly_sparse_decode_attn and tq_vonly_decode_step_at refuse it (UNSUPPORTED), and nothing is
    written by a refused call."""
    from tqhip import ops
    B, n_kv, n_rep, T, D = 1, 2, 7, 700, 128
    n_q = n_kv * n_rep
    sc = 1 / math.sqrt(D)
    c = tq.VOnlyTurboQuantCache(bits=3, fused=True)
    c.update_and_fetch(rand((B, n_kv, T, D), 1700), rand((B, n_kv, T, D), 1701))
    kc, vt = c._k_cache, c._v_tq
    K, vp, vn = kc.keys[:, :, :T], vt.v_packed[:, :, :T], vt.v_norms[:, :, :T]
    cb, sg = vt._v_q.centroids, vt._v_q.signs
    q = rand((B, n_q, D), 1702, qdt)
    q_off = _offset_view(q)
    want = tq.vonly_decode(q, K, vp, vn, cb, sg, D, 3, sc, n_rep=n_rep, seq_len=T)
    got = tq.vonly_decode(q_off, K, vp, vn, cb, sg, D, 3, sc, n_rep=n_rep, seq_len=T)
    assert bool(((got - want).abs() <= 1e-3 + 2e-3 * want.abs()).all())
    fp32 = tq.vonly_decode(q, K, vp, vn, cb, sg, D, 3, sc, n_rep=n_rep, seq_len=T, precision="fp32")
    assert torch.equal(got, fp32), "a q off the boundary is served by the float32 kernels"
    out = torch.full((B, n_q, D), 7.0, device="cuda")
    with pytest.raises(RuntimeError, match="aligned q"):
        tq.vonly_decode(q_off, K, vp, vn, cb, sg, D, 3, sc, n_rep=n_rep, seq_len=T, sparse_v_threshold=1e-5, out=out)
    torch.cuda.synchronize()
    assert bool((out == 7.0).all())
    # the single-call step: host position -> two-call route, device position -> refused
    k1, v1 = rand((B, n_kv, D), 1703), rand((B, n_kv, D), 1704)
    twin = tq.VOnlyTurboQuantCache(bits=3, fused=True)
    twin.update_and_fetch(rand((B, n_kv, T, D), 1700), rand((B, n_kv, T, D), 1701))
    a = c.decode_step(q.view(B, n_q, 1, D), k1.view(B, n_kv, 1, D), v1.view(B, n_kv, 1, D), sc)
    b = twin.decode_step(q_off.view(B, n_q, 1, D), k1.view(B, n_kv, 1, D), v1.view(B, n_kv, 1, D), sc)
    assert bool(((a.float() - b.float()).abs() <= 1e-3 + 2e-3 * a.float().abs()).all())
    for x, y in zip(c.state, twin.state):
        assert torch.equal(x, y)
    pos = torch.tensor([c.offset], dtype=torch.int64, device="cuda")
    c.reserve(B, n_kv, 4, D)
    before = [t.clone() for t in c.state]
    with pytest.raises(RuntimeError, match="aligned q"):
        c.decode_step(q_off.view(B, n_q, 1, D), k1.view(B, n_kv, 1, D), v1.view(B, n_kv, 1, D), sc, position=pos,
                      out=torch.empty((B, n_q, 1, D), dtype=q.dtype, device="cuda"))
    torch.cuda.synchronize()
    for x, y in zip(c.state, before):
        assert torch.equal(x, y)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_packed_cache_decode_step_is_update_plus_attention(tq, dtype):
    """TurboQuantKVCache.decode_step (tq_packed_decode_step: the tile pass over the old positions + a merge pass
    that encodes both new rows, scores the new key and stores them) agrees, step after step and across a growth
    of the storage, with update_and_fetch + turboquant_attention(fused=True) on a twin cache to the 2e-3 / 1e-3
    bar, leaves the very same state behind, and its output matches the float64 oracle; a d = 64 cache takes the
    two-call route and agrees bit for bit."""
    B, n_q, n_kv, D, S0 = 2, 32, 8, 128, 250
    sc = 1 / math.sqrt(D)
    k0, v0 = rand((B, n_kv, S0, D), 800, dtype), rand((B, n_kv, S0, D), 801, dtype)
    a, b = tq.TurboQuantKVCache(bits=3, fused=True), tq.TurboQuantKVCache(bits=3, fused=True)
    a.update_and_fetch(k0, v0), b.update_and_fetch(k0, v0)
    for i in range(9):                                              # 250 -> 259: grows at 256
        k1, v1, q1 = rand((B, n_kv, 1, D), 810 + 3 * i, dtype), rand((B, n_kv, 1, D), 811 + 3 * i, dtype), rand((B, n_q, 1, D), 812 + 3 * i, dtype)
        got = a.decode_step(q1, k1, v1, sc)
        b.update_and_fetch(k1, v1)
        want = tq.turboquant_attention(q1, b, sc, fused=True)
        assert got.shape == (B, n_q, 1, D) and got.dtype == dtype
        err = (got.float() - want.float()).abs()
        bar = 1e-3 + (2e-3 if dtype == torch.float16 else 8e-3) * want.float().abs()    # bf16 outputs: one ulp is 2^-8
        assert bool((err <= bar).all()), (i, float(err.max()))
    assert a.offset == b.offset == S0 + 9 and a.v_packed.shape[2] == 512
    for x, y in zip(a.state, b.state):
        assert torch.equal(x, y)
    kp, kn, vp, vn = [t.cpu().numpy() for t in a.state]
    kq, vq = a._k_q, a._v_q
    for s in range(B):
        ref = o.turboquant_attention_single(host(q1[s, :, 0]), kp[s].view(np.uint32), kn[s], vp[s].view(np.uint32), vn[s],
                                            np.asarray(kq.centroids.cpu()), kq.signs.cpu().numpy(),
                                            np.asarray(vq.centroids.cpu()), vq.signs.cpu().numpy(), D, 3, sc)
        err = np.abs(host(got[s, :, 0]).astype(np.float64) - ref)
        tol = 1e-3 + (2e-3 if dtype == torch.float16 else 6e-3) * np.abs(ref)
        assert (err <= tol).all(), err.max()
    c4, d4 = tq.TurboQuantKVCache(bits=3, fused=True), tq.TurboQuantKVCache(bits=3, fused=True)
    k0, v0, k1, v1, q1 = k0[..., :64], v0[..., :64], k1[..., :64], v1[..., :64], q1[..., :64]
    c4.update_and_fetch(k0, v0), d4.update_and_fetch(k0, v0)
    got = c4.decode_step(q1, k1, v1, sc)
    d4.update_and_fetch(k1, v1)
    assert torch.equal(got, tq.turboquant_attention(q1, d4, sc, fused=True)) and c4.offset == d4.offset


def test_vonly_decode_step_replayed_from_a_hip_graph(tq):
    """A decode step recorded ONCE in a HIP graph with the position held in device memory
    (tq_vonly_decode_step_at) and replayed for ten tokens, with eager work and synchronisations between the
    replays: every replay matches the eager step on a twin cache and the float64 oracle, and the two caches
    end in the same state bit for bit.  An insert past the storage is dropped."""
    B, n_q, n_kv, D, S0, N = 2, 28, 4, 128, 300, 10
    sc = 1 / math.sqrt(D)
    k0, v0 = rand((B, n_kv, S0, D), 900), rand((B, n_kv, S0, D), 901)
    cg, ce = tq.VOnlyTurboQuantCache(bits=3, fused=True), tq.VOnlyTurboQuantCache(bits=3, fused=True)
    cg.reserve(B, n_kv, 1024, D)
    cg.update_and_fetch(k0, v0), ce.update_and_fetch(k0, v0)
    t_alloc = cg._k_cache.keys.shape[2]
    assert t_alloc == 1024 and cg._v_tq.v_packed.shape[2] == 1024
    pos = torch.tensor([S0], dtype=torch.int64, device="cuda")
    qs, ks, vs = rand((B, n_q, 1, D), 902), rand((B, n_kv, 1, D), 903), rand((B, n_kv, 1, D), 904)
    out_s = torch.empty((B, n_q, D), dtype=torch.float16, device="cuda")

    def check(step_no, q, k, v):
        want = ce.decode_step(q, k, v, sc)
        got = out_s.clone()
        err = (got.float() - want[:, :, 0].float()).abs()
        assert bool((err <= 1e-3 + 2e-3 * want[:, :, 0].float().abs()).all()), (step_no, float(err.max()))
        return got

    cg.decode_step(qs, ks, vs, sc, position=pos, out=out_s)          # eager once: workspace, descriptor
    pos.add_(1)
    check(-1, qs, ks, vs)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        cg.decode_step(qs, ks, vs, sc, position=pos, out=out_s)
        pos.add_(1)
    for i in range(N):
        q, k, v = rand((B, n_q, 1, D), 910 + 3 * i), rand((B, n_kv, 1, D), 911 + 3 * i), rand((B, n_kv, 1, D), 912 + 3 * i)
        qs.copy_(q), ks.copy_(k), vs.copy_(v)
        graph.replay()
        got = check(i, q, k, v)
        torch.cuda.synchronize()
        assert int(pos.item()) == S0 + 2 + i
    cg.set_offset(S0 + 1 + N)
    assert cg.offset == ce.offset == S0 + 1 + N
    for x, y in zip(cg.state, ce.state):
        assert torch.equal(x, y)
    st = cg.state
    vq = cg._v_tq._v_q
    for s_ in range(B):
        ref = o.vonly_decode_attention(host(q[s_, :, 0]), st[0][s_].cpu().numpy(), st[2][s_].cpu().numpy().view(np.uint32),
                                       st[3][s_].cpu().numpy(), np.asarray(vq.centroids.cpu()), vq.signs.cpu().numpy(), D, 3, sc)
        err = np.abs(host(got[s_]).astype(np.float64) - ref)
        assert (err <= 1e-3 + 2e-3 * np.abs(ref)).all(), err.max()
    # past the storage: nothing is written, the step still runs
    before = [t.clone() for t in (cg._k_cache.keys, cg._v_tq.v_packed, cg._v_tq.v_norms)]
    pos.fill_(t_alloc)
    graph.replay()
    torch.cuda.synchronize()
    for x, y in zip(before, (cg._k_cache.keys, cg._v_tq.v_packed, cg._v_tq.v_norms)):
        assert torch.equal(x, y)
    assert bool(torch.isfinite(out_s.float()).all())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_vonly_decode_step_from_an_empty_cache_and_at_tile_boundaries(tq, dtype):
    """The merge pass that inserts the token: from an empty cache (no tile pass at all: the output is the
    dequantised new value), and at lengths around the 256- and 512-position tile boundaries, with keys, values
    and queries of every dtype; the state equals the two-call cache's bit for bit (the encoder's arithmetic is
    restated there operation for operation) and the output matches the float64 oracle."""
    B, n_q, n_kv, D = 2, 8, 2, 128
    sc = 1 / math.sqrt(D)
    a, b = tq.VOnlyTurboQuantCache(bits=3, fused=True), tq.VOnlyTurboQuantCache(bits=3, fused=True)
    vq = None
    seed = 1000
    for grow in (0, 254, 255, 2, 253, 1):                           # steps at lengths 0, 255, 511, 512, 513, 767, 768, 769
        if grow:
            k0, v0 = rand((B, n_kv, grow, D), seed, dtype), rand((B, n_kv, grow, D), seed + 1, dtype)
            a.update_and_fetch(k0, v0), b.update_and_fetch(k0, v0)
        for _ in range(2 if grow in (2, 1) else 1):
            seed += 5
            k1, v1, q1 = rand((B, n_kv, 1, D), seed + 2, dtype), rand((B, n_kv, 1, D), seed + 3, dtype), rand((B, n_q, 1, D), seed + 4, dtype)
            got = a.decode_step(q1, k1, v1, sc)
            b.update_and_fetch(k1, v1)
            assert a.offset == b.offset
            st = a.state
            for x, y in zip(st, b.state):
                assert x.dtype == y.dtype and torch.equal(x, y), a.offset
            vq = a._v_tq._v_q
            for s_ in range(B):
                ref = o.vonly_decode_attention(host(q1[s_, :, 0]), st[0][s_].cpu().numpy(), st[2][s_].cpu().numpy().view(np.uint32),
                                               st[3][s_].cpu().numpy(), np.asarray(vq.centroids.cpu()), vq.signs.cpu().numpy(), D, 3, sc)
                err = np.abs(host(got[s_, :, 0]).astype(np.float64) - ref)
                tol = 1e-3 + (8e-3 if dtype == torch.bfloat16 else 2e-3) * np.abs(ref)
                assert (err <= tol).all(), (a.offset, err.max())
    assert a.offset == 0 + 1 + 254 + 1 + 255 + 1 + 2 + 2 + 253 + 1 + 1 + 2


def test_vonly_decode_step_other_shapes_take_the_append_route(tq):
    """d = 64: tq_vonly_decode_step has no two-launch form there and runs tq_vonly_append +
    tq_vonly_decode_attn inside the one call: the very bits of the two calls of the Python surface."""
    B, n_q, n_kv, D, S0 = 1, 6, 2, 64, 70
    sc = 1 / math.sqrt(D)
    a, b = tq.VOnlyTurboQuantCache(bits=4, fused=True), tq.VOnlyTurboQuantCache(bits=4, fused=True)
    k0, v0 = rand((B, n_kv, S0, D), 1100), rand((B, n_kv, S0, D), 1101)
    a.update_and_fetch(k0, v0), b.update_and_fetch(k0, v0)
    for i in range(3):
        k1, v1, q1 = rand((B, n_kv, 1, D), 1110 + 3 * i), rand((B, n_kv, 1, D), 1111 + 3 * i), rand((B, n_q, 1, D), 1112 + 3 * i)
        got = a.decode_step(q1, k1, v1, sc)
        b.update_and_fetch(k1, v1)
        assert torch.equal(got, tq.vonly_decode_attention(q1, b, sc))
    for x, y in zip(a.state, b.state):
        assert torch.equal(x, y)
    pos = torch.tensor([a.offset], dtype=torch.int64, device="cuda")
    with pytest.raises((ValueError, RuntimeError)):
        a.decode_step(q1, k1, v1, sc, position=pos)                  # the device-side position needs d = 128


@pytest.mark.parametrize("S0,want_alloc", [(300, 1024), (31000, 32768)])
def test_packed_decode_step_replayed_from_a_hip_graph(tq, S0, want_alloc):
    """The packed cache's decode step recorded once in a HIP graph with the position in device memory
    (tq_packed_decode_step_at) and replayed for eight tokens, with eager work and synchronisations between
    the replays: every replay matches the eager step on a twin cache, and both caches end in the same state
    bit for bit.  An insert past the storage is dropped.  The long case runs the streaming pass (storage of
    32768 positions x 8 kv heads), the short one the single-tile pass."""
    B, n_q, n_kv, D, N = 1, 32, 8, 128, 8
    sc = 1 / math.sqrt(D)
    k0, v0 = rand((B, n_kv, S0, D), 1200), rand((B, n_kv, S0, D), 1201)
    cg, ce = tq.TurboQuantKVCache(bits=3, fused=True), tq.TurboQuantKVCache(bits=3, fused=True)
    cg.reserve(B, n_kv, want_alloc, D)
    cg.update_and_fetch(k0, v0), ce.update_and_fetch(k0, v0)
    t_alloc = cg.v_packed.shape[2]
    assert t_alloc == want_alloc
    from tqhip import _lib
    assert (_lib.load().tq_flash_decode_plan(B, n_kv, t_alloc, 1, 0) >= 2) == (want_alloc == 32768)
    pos = torch.tensor([S0], dtype=torch.int64, device="cuda")
    qs, ks, vs = rand((B, n_q, 1, D), 1202), rand((B, n_kv, 1, D), 1203), rand((B, n_kv, 1, D), 1204)
    out_s = torch.empty((B, n_q, D), dtype=torch.float16, device="cuda")

    def check(step_no, q, k, v):
        want = ce.decode_step(q, k, v, sc)[:, :, 0].float()
        err = (out_s.float() - want).abs()
        assert bool((err <= 1e-3 + 2e-3 * want.abs()).all()), (step_no, float(err.max()))

    cg.decode_step(qs, ks, vs, sc, position=pos, out=out_s)
    pos.add_(1)
    check(-1, qs, ks, vs)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        cg.decode_step(qs, ks, vs, sc, position=pos, out=out_s)
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


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_packed_decode_step_from_an_empty_cache_and_at_a_tile_boundary(tq, dtype):
    """The packed cache's in-merge insert from an empty cache (no tile pass) and around the 512-position tile
    boundary: state bit-identical to the two-call cache, output against the float64 oracle."""
    B, n_q, n_kv, D = 2, 8, 2, 128
    sc = 1 / math.sqrt(D)
    a, b = tq.TurboQuantKVCache(bits=3, fused=True), tq.TurboQuantKVCache(bits=3, fused=True)
    seed = 1300
    for grow in (0, 509, 0, 0):                                     # steps at lengths 0, 510, 511, 512
        if grow:
            k0, v0 = rand((B, n_kv, grow, D), seed, dtype), rand((B, n_kv, grow, D), seed + 1, dtype)
            a.update_and_fetch(k0, v0), b.update_and_fetch(k0, v0)
        seed += 5
        k1, v1, q1 = rand((B, n_kv, 1, D), seed + 2, dtype), rand((B, n_kv, 1, D), seed + 3, dtype), rand((B, n_q, 1, D), seed + 4, dtype)
        got = a.decode_step(q1, k1, v1, sc)
        b.update_and_fetch(k1, v1)
        assert a.offset == b.offset
        for x, y in zip(a.state, b.state):
            assert torch.equal(x, y), a.offset
        kp, kn, vp, vn = [t.cpu().numpy() for t in a.state]
        kq, vq = a._k_q, a._v_q
        for s_ in range(B):
            ref = o.turboquant_attention_single(host(q1[s_, :, 0]), kp[s_].view(np.uint32), kn[s_], vp[s_].view(np.uint32), vn[s_],
                                                np.asarray(kq.centroids.cpu()), kq.signs.cpu().numpy(),
                                                np.asarray(vq.centroids.cpu()), vq.signs.cpu().numpy(), D, 3, sc)
            err = np.abs(host(got[s_, :, 0]).astype(np.float64) - ref)
            assert (err <= 1e-3 + 2e-3 * np.abs(ref)).all(), (a.offset, err.max())
    assert a.offset == 513


def test_vonly_append_with_a_device_side_position(tq):
    """tq_vonly_append_at: three tokens inserted at a position held in device memory give the storage of the
    host-position call bit for bit; rows that would land past the storage are dropped, the others kept."""
    from tqhip import ops
    B, H, T, S, D = 2, 3, 64, 3, 128
    sg = o.random_diagonal_sign(D, 43)
    signs = torch.from_numpy(sg).cuda()
    c = o.gaussian_codebook(3)
    bnd = o.gaussian_boundaries(c)
    k, v = rand((B, H, S, D), 1400, torch.bfloat16), rand((B, H, S, D), 1401)

    def storage():
        return (torch.zeros((B, H, T, D), dtype=torch.float16, device="cuda"), torch.zeros((B, H, T, D), dtype=torch.float16, device="cuda"),
                torch.zeros((B, H, T, 13), dtype=torch.int32, device="cuda").view(torch.uint32), torch.zeros((B, H, T), device="cuda"))
    for pos in (17, T - 2):
        a, b = storage(), storage()
        n_fit = min(S, T - pos)
        ops.vonly_append_into(k[:, :, :n_fit], v[:, :, :n_fit], signs, bnd, a[0], a[1], a[2], a[3], position=pos, bits=3)
        ops.vonly_append_into(k, v, signs, bnd, b[0], b[1], b[2], b[3],
                              position=torch.tensor([pos], dtype=torch.int64, device="cuda"), bits=3)
        for x, y in zip(a, b):
            assert torch.equal(x, y), pos
        assert float(a[3][:, :, pos:pos + n_fit].min()) > 0.0


def test_decode_step_after_from_state_and_trim(tq):
    """decode_step on caches rebuilt with from_state (storage handed in as slices, possibly of unequal
    allocated lengths) and after trim: same state as the two calls, output within the bar."""
    B, n_q, n_kv, D, S0 = 1, 8, 2, 128, 300
    sc = 1 / math.sqrt(D)
    k0, v0 = rand((B, n_kv, S0, D), 1500), rand((B, n_kv, S0, D), 1501)
    for make, attend in ((lambda: tq.VOnlyTurboQuantCache(bits=3, fused=True), tq.vonly_decode_attention),
                         (lambda: tq.TurboQuantKVCache(bits=3, fused=True), lambda q, c, s: tq.turboquant_attention(q, c, s, fused=True))):
        src = make()
        src.update_and_fetch(k0, v0)
        a = type(src).from_state(src.state, src.meta_state)
        b = type(src).from_state(src.state, src.meta_state)
        a.fused = b.fused = True
        a.trim(7), b.trim(7)
        for i in range(3):
            k1, v1, q1 = rand((B, n_kv, 1, D), 1510 + 3 * i), rand((B, n_kv, 1, D), 1511 + 3 * i), rand((B, n_q, 1, D), 1512 + 3 * i)
            got = a.decode_step(q1, k1, v1, sc)
            b.update_and_fetch(k1, v1)
            want = attend(q1, b, sc)
            err = (got.float() - want.float()).abs()
            assert bool((err <= 1e-3 + 2e-3 * want.float().abs()).all()), float(err.max())
        assert a.offset == b.offset == S0 - 7 + 3
        for x, y in zip(a.state, b.state):
            assert torch.equal(x, y)


# ------------------------------------------------------------------ explicit sign vectors

def _pm1(dim, seed):
    rng = np.random.default_rng(seed)
    return np.where(rng.random(dim) < 0.5, -1.0, 1.0).astype(F32)


def test_packed_cache_with_explicit_signs_round_trips(tq):
    """A cache built with caller-supplied sign vectors (cache.py:33-39,90-98 take them from the seed): packed
    state equals the oracle's for THOSE signs, differs from the seed-derived one, survives state / meta_state /
    from_state(..., k_signs, v_signs) bit for bit, and attends within the bar both before and after."""
    B, n_q, n_kv, D, S = 1, 8, 2, 128, 300
    sc = 1 / math.sqrt(D)
    ks, vs = _pm1(D, 901), _pm1(D, 902)
    k, v = rand((B, n_kv, S, D), 910), rand((B, n_kv, S, D), 911)
    q = rand((B, n_q, 1, D), 912)
    c = tq.TurboQuantKVCache(bits=3, fused=True, k_signs=ks, v_signs=torch.from_numpy(vs))
    c.update_and_fetch(k, v)
    cb = o.gaussian_codebook(3)
    bd = o.gaussian_boundaries(cb)
    kp, kn = o.fused_quantize(host(k).reshape(-1, D), ks, bd, D, 3)
    vp, vn = o.fused_quantize(host(v).reshape(-1, D), vs, bd, D, 3)
    assert np.array_equal(c.k_packed[..., :S, :].cpu().numpy().reshape(-1, 13), kp)
    assert np.array_equal(c.v_packed[..., :S, :].cpu().numpy().reshape(-1, 13), vp)
    assert np.array_equal(c.k_norms[..., :S].cpu().numpy().ravel(), kn)
    seeded = tq.TurboQuantKVCache(bits=3, fused=True)
    seeded.update_and_fetch(k, v)
    assert not torch.equal(seeded.k_packed, c.k_packed)
    want = np.stack([o.flash_attention_turboquant(
        o.prerotate_query(host(q)[0, :, 0, :], ks), kp.reshape(n_kv, S, 13), kn.reshape(n_kv, S), vp.reshape(n_kv, S, 13),
        vn.reshape(n_kv, S), cb, cb, vs, D, 3, n_rep=n_q // n_kv, attn_scale=sc)])
    got = host(tq.turboquant_attention(q, c, sc, fused=True))[:, :, 0, :]
    err = np.abs(got - want)
    assert np.all(err <= 1e-3 + 2e-3 * np.abs(want)), err.max()
    # serialise and restore: with the signs the restored cache is the same cache
    r = tq.TurboQuantKVCache.from_state([t.clone() for t in c.state], c.meta_state, k_signs=ks, v_signs=vs)
    for x, y in zip(r.state, c.state):
        assert torch.equal(x, y)
    assert r.meta_state == c.meta_state
    got_r = host(tq.turboquant_attention(q, r, sc, fused=True))[:, :, 0, :]
    assert np.array_equal(got_r, got)
    # ... and can extend: the new rows are encoded with the given signs
    k1, v1 = rand((B, n_kv, 5, D), 913), rand((B, n_kv, 5, D), 914)
    r.fused = True
    r.update_and_fetch(k1, v1)
    kp1, _ = o.fused_quantize(host(k1).reshape(-1, D), ks, bd, D, 3)
    assert np.array_equal(r.k_packed[..., S:S + 5, :].cpu().numpy().reshape(-1, 13), kp1)
    # without the signs the restored cache decodes with the seed's vector: a different (wrong) result
    wrong = tq.TurboQuantKVCache.from_state([t.clone() for t in c.state], c.meta_state)
    got_w = host(tq.turboquant_attention(q, wrong, sc, fused=True))[:, :, 0, :]
    assert np.abs(got_w - want).max() > 0.05
    with pytest.raises(ValueError):
        tq.TurboQuantKVCache(bits=3, k_signs=np.ones(64, F32)).update_and_fetch(k, v)
    with pytest.raises(ValueError):
        tq.TurboQuantKVCache(bits=3, v_signs=np.zeros(D, F32)).update_and_fetch(k, v)


def test_vonly_cache_with_explicit_signs_round_trips(tq):
    """VOnlyTurboQuantCache(v_signs=...) and from_state(..., v_signs=...): values dequantise to the oracle's for
    those signs, the restored cache is bit-identical and attends like the original."""
    B, n_q, n_kv, D, S = 1, 14, 2, 128, 260
    sc = 1 / math.sqrt(D)
    vs = _pm1(D, 921)
    k, v = rand((B, n_kv, S, D), 930), rand((B, n_kv, S, D), 931)
    q = rand((B, n_q, 1, D), 932)
    c = tq.VOnlyTurboQuantCache(bits=3, v_signs=vs)
    _, v_deq = c.update_and_fetch(k, v)
    cb = o.gaussian_codebook(3)
    vp, vn = o.fused_quantize(host(v).reshape(-1, D), vs, o.gaussian_boundaries(cb), D, 3)
    assert np.array_equal(c._v_tq.v_packed[..., :S, :].cpu().numpy().reshape(-1, 13), vp)
    want_deq = o.packed_dequantize(vp, vn, cb, vs, D, 3).reshape(B, n_kv, S, D)
    assert np.abs(host(v_deq) - want_deq).max() <= 2e-3           # fp16 output of exact float32 values
    want = o.vonly_decode_attention(host(q)[0, :, 0, :], host(k)[0].astype(np.float16), vp.reshape(n_kv, S, 13),
                                    vn.reshape(n_kv, S), cb, vs, D, 3, sc)
    got = host(tq.vonly_decode_attention(q, c, sc))[0, :, 0, :]
    assert np.all(np.abs(got - want) <= 1e-3 + 2e-3 * np.abs(want))
    r = tq.VOnlyTurboQuantCache.from_state([t.clone() for t in c.state], c.meta_state, v_signs=vs)
    assert r.offset == S and r.meta_state == c.meta_state
    for x, y in zip(r.state, c.state):
        assert torch.equal(x, y)
    assert np.array_equal(host(tq.vonly_decode_attention(q, r, sc))[0, :, 0, :], got)
    k1, v1, q1 = rand((B, n_kv, 1, D), 933), rand((B, n_kv, 1, D), 934), rand((B, n_q, 1, D), 935)
    o1 = host(r.decode_step(q1, k1, v1, sc))[0, :, 0, :]
    c.update_and_fetch(k1, v1)
    o2 = host(tq.vonly_decode_attention(q1, c, sc))[0, :, 0, :]
    assert np.all(np.abs(o1 - o2) <= 1e-3 + 2e-3 * np.abs(o2))
    for x, y in zip(r.state, c.state):
        assert torch.equal(x, y)


# ------------------------------------------------------------------ one capacity for keys and values

def _vonly_filled(tq, chunks, seed, **kw):
    B, n_kv, D = 1, 2, 128
    c = tq.VOnlyTurboQuantCache(bits=3, **kw)
    for i, S in enumerate(chunks):
        c.update_and_fetch(rand((B, n_kv, S, D), seed + 2 * i), rand((B, n_kv, S, D), seed + 2 * i + 1))
    return c


@pytest.mark.parametrize("chunks,fused", [((1000,), False), ((1000, 500), False), ((1000,), True), ((700, 300, 3), True)])
def test_vonly_single_call_step_after_real_prompts(tq, chunks, fused):
    """A prompt through update_and_fetch leaves the key cache and the packed values with different capacities
    (they grow by different rules); reserve() and decode_step() must bring them to one capacity so that the
    single-call step (host position AND device-side position) runs on its descriptor, not on the two-call
    fallback: the descriptor is asserted to exist, results and state are compared with the two calls."""
    B, n_q, n_kv, D = 1, 14, 2, 128
    sc = 1 / math.sqrt(D)
    a = _vonly_filled(tq, chunks, 1700, fused=fused)
    b = _vonly_filled(tq, chunks, 1700, fused=True)
    n0 = sum(chunks)
    a.reserve(B, n_kv, 2000, D)
    assert a._k_cache.keys.shape[2] == a._v_tq.v_packed.shape[2] >= n0 + 2000
    assert a._k_cache.keys.shape[2] % 256 == 0
    for x, y in zip(a.state, b.state):
        assert torch.equal(x, y)
    pos = torch.tensor([n0], dtype=torch.int64, device="cuda")
    out = torch.empty((B, n_q, D), dtype=torch.float16, device="cuda")
    for i in range(3):
        k1, v1, q1 = rand((B, n_kv, 1, D), 1710 + 3 * i), rand((B, n_kv, 1, D), 1711 + 3 * i), rand((B, n_q, 1, D), 1712 + 3 * i)
        if i < 2:
            a.decode_step(q1, k1, v1, sc, position=pos, out=out)
            pos.add_(1)
            got = out.clone()[:, :, None, :]
        else:
            a.set_offset(int(pos.item()))
            got = a.decode_step(q1, k1, v1, sc)
        assert a._step is not None and a._step.shape[2] == a._k_cache.keys.shape[2], "the two-call fallback ran"
        b.update_and_fetch(k1, v1)
        want = tq.vonly_decode_attention(q1, b, sc)
        err = (got.float() - want.float()).abs()
        assert bool((err <= 1e-3 + 2e-3 * want.float().abs()).all()), float(err.max())
    assert a.offset == b.offset == n0 + 3
    for x, y in zip(a.state, b.state):
        assert torch.equal(x, y)


def test_vonly_single_call_step_after_from_state(tq):
    """from_state hands the storage in as slices (300 positions; the key cache would grow to 556, the packed
    values to 512): the first decode_step realigns both to one contiguous capacity and runs on the descriptor,
    also with a device-side position."""
    B, n_q, n_kv, D, S0 = 1, 8, 2, 128, 300
    sc = 1 / math.sqrt(D)
    src = _vonly_filled(tq, (S0,), 1800, fused=True)
    a = tq.VOnlyTurboQuantCache.from_state(src.state, src.meta_state)
    a.fused = True
    a.reserve(B, n_kv, 1, D)
    assert a._k_cache.keys.shape[2] == a._v_tq.v_packed.shape[2] == 512 and a._k_cache.keys.is_contiguous()
    pos = torch.tensor([S0], dtype=torch.int64, device="cuda")
    for i in range(2):
        k1, v1, q1 = rand((B, n_kv, 1, D), 1810 + 3 * i), rand((B, n_kv, 1, D), 1811 + 3 * i), rand((B, n_q, 1, D), 1812 + 3 * i)
        got = a.decode_step(q1, k1, v1, sc, position=pos)
        pos.add_(1)
        assert a._step is not None
        src.update_and_fetch(k1, v1)
        want = tq.vonly_decode_attention(q1, src, sc)
        err = (got.float() - want.float()).abs()
        assert bool((err <= 1e-3 + 2e-3 * want.float().abs()).all()), float(err.max())
    a.set_offset(int(pos.item()))
    for x, y in zip(a.state, src.state):
        assert torch.equal(x, y)
    with pytest.raises(ValueError):
        a.set_offset(513)


def test_step_descriptor_keeps_its_workspace_alive(tq):
    """The workspace address goes into every call of a step descriptor (and into a HIP graph that records one).
    When a later, larger op replaces the shared per-stream workspace, the descriptor must still hold the buffer
    it used: its graph replays keep writing there."""
    from tqhip import ops
    B, n_q, n_kv, D = 1, 14, 2, 128
    sc = 1 / math.sqrt(D)
    a = _vonly_filled(tq, (600,), 1900, fused=True)
    b = _vonly_filled(tq, (600,), 1900, fused=True)
    a.reserve(B, n_kv, 64, D)
    pos = torch.tensor([600], dtype=torch.int64, device="cuda")
    ks, vs_, qs = rand((B, n_kv, 1, D), 1910), rand((B, n_kv, 1, D), 1911), rand((B, n_q, 1, D), 1912)
    out = torch.empty((B, n_q, D), dtype=torch.float16, device="cuda")
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        a.decode_step(qs, ks, vs_, sc, position=pos, out=out)      # warm-up on the capture stream
        side.synchronize()
        first_ws = a._step._ws
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            a.decode_step(qs, ks, vs_, sc, position=pos, out=out)
    torch.cuda.synchronize()
    key = (first_ws.device, side.cuda_stream)
    assert ops._workspaces[key] is first_ws
    with torch.cuda.stream(side):                                  # a larger request on that stream replaces the shared buffer
        ops._workspace(first_ws.device, side.cuda_stream, first_ws.numel() * 4 + 1)
    assert ops._workspaces[key] is not first_ws
    assert any(w is first_ws for w in a._step._ws_refs), "the descriptor dropped the workspace its graph writes to"
    filler = torch.full((first_ws.numel() * 2,), 7, dtype=torch.uint8, device="cuda")   # would land in freed memory
    for i in range(3):
        g.replay()
        torch.cuda.synchronize()
        pos.add_(1)
        torch.cuda.synchronize()
        b.update_and_fetch(ks, vs_)
        want = tq.vonly_decode_attention(qs, b, sc)[:, :, 0, :]
        err = (out.float() - want.float()).abs()
        assert bool((err <= 1e-3 + 2e-3 * want.float().abs()).all()), (i, float(err.max()))
    assert int(filler.sum()) == 7 * filler.numel()
