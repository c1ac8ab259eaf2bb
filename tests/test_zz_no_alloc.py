"""The entry point that allocates nothing: tq_vonly_decode_attn_static keeps its per-tile partial sums in an
array inside the library instead of a caller's workspace.  Called through the C ABI and compared with
tq_vonly_decode_attn (same kernels, so bit-identical output is the bar) on two calls in a row, the second
with a smaller input, and against the oracle; torch's allocator must not be touched by the call itself.
This file sorts after the other test files on purpose: pytest stops at the first failure.
"""
import ctypes as C
import math

import numpy as np
import pytest

torch = pytest.importorskip("torch")

from oracle import polarquant_oracle as o  # noqa: E402

pytestmark = pytest.mark.gpu

D, BITS = 128, 3


def _case(tq, rng, n_seq, n_kv, n_rep, T, q_dtype=np.float16):
    c = o.gaussian_codebook(BITS)
    b = o.gaussian_boundaries(c)
    vs = o.random_diagonal_sign(D, 43)
    K = rng.standard_normal((n_seq, n_kv, T, D)).astype(np.float16)
    V = rng.standard_normal((n_seq * n_kv * T, D)).astype(np.float16)
    q = rng.standard_normal((n_seq, n_kv * n_rep, D)).astype(q_dtype)
    vp, vn = tq.fused_quantize(torch.from_numpy(V).cuda(), torch.from_numpy(vs).cuda(), b, D, BITS)
    return dict(q=torch.from_numpy(q).cuda(), K=torch.from_numpy(K).cuda(), vp=vp.reshape(n_seq, n_kv, T, -1),
                vn=vn.reshape(n_seq, n_kv, T), c=c, vs=torch.from_numpy(vs).cuda(), n_rep=n_rep, T=T,
                q_np=q, K_np=K, vs_np=vs)


def _both(tq, case, out_dtype=torch.float32):
    """(static-scratch result, workspace result): the first written into a preallocated tensor."""
    sc = 1.0 / math.sqrt(D)
    n_seq, n_q, _ = case["q"].shape
    out = torch.full((n_seq, n_q, D), float("nan"), dtype=out_dtype, device="cuda")
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    got = tq.vonly_decode(case["q"], case["K"], case["vp"], case["vn"], case["c"], case["vs"], D, BITS, sc,
                          n_rep=case["n_rep"], out=out, static_scratch=True)
    after = torch.cuda.memory_stats()["allocation.all.allocated"]
    assert got is out
    assert after == before, "the static-scratch call allocated device memory through torch"
    want = tq.vonly_decode(case["q"], case["K"], case["vp"], case["vn"], case["c"], case["vs"], D, BITS, sc,
                           n_rep=case["n_rep"], out_dtype=out_dtype)
    torch.cuda.synchronize()
    return got, want


@pytest.fixture(scope="module")
def tq():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a GPU: torch.cuda.is_available() is False")
    import tqhip
    return tqhip


def test_static_scratch_two_calls_second_smaller(tq):
    """Config-2 heads at 8192 positions, then 1000 positions (a ragged last tile, fewer tiles than the first
    call left partial sums for): both bit-identical to the workspace entry point and inside 2e-3 / 1e-3 of
    the oracle."""
    rng = np.random.default_rng(7)
    sc = 1.0 / math.sqrt(D)
    for T in (8192, 1000):
        case = _case(tq, rng, 1, 4, 7, T)
        got, want = _both(tq, case)
        assert torch.equal(got, want), f"T={T}: static-scratch output differs from tq_vonly_decode_attn"
        vp, vn = case["vp"].cpu().numpy()[0], case["vn"].cpu().numpy()[0]
        ref = o.vonly_decode_attention(case["q_np"][0], case["K_np"][0], vp, vn, case["c"], case["vs_np"], D, BITS, sc)
        err = np.abs(got[0].cpu().numpy() - ref)
        assert np.all(err <= 1e-3 + 2e-3 * np.abs(ref)), f"T={T}: off the oracle by {err.max():.3e}"


def test_static_scratch_batch_dtypes_and_float32_path(tq):
    """A batch of 3 sequences with fp16 output, float32 queries (fp16 value + remainder kernels), and the float32
    vector-ALU kernels (precision='fp32' shares the entry point): each bit-identical to the workspace call."""
    rng = np.random.default_rng(8)
    sc = 1.0 / math.sqrt(D)
    case = _case(tq, rng, 3, 2, 4, 777)
    got, want = _both(tq, case, out_dtype=torch.float16)
    assert torch.equal(got, want)
    case = _case(tq, rng, 1, 2, 7, 300, q_dtype=np.float32)
    got, want = _both(tq, case)
    assert torch.equal(got, want)
    out = torch.empty((1, 14, D), dtype=torch.float32, device="cuda")
    a = tq.vonly_decode(case["q"], case["K"], case["vp"], case["vn"], case["c"], case["vs"], D, BITS, sc, n_rep=7,
                        precision="fp32", out=out, static_scratch=True)
    b = tq.vonly_decode(case["q"], case["K"], case["vp"], case["vn"], case["c"], case["vs"], D, BITS, sc, n_rep=7,
                        precision="fp32")
    assert torch.equal(a, b)


def test_static_scratch_leaves_device_memory_alone_and_replays_from_a_graph(tq):
    """The driver's own count of free device memory (hipMemGetInfo) is the same before and after a run of
    calls -- torch's allocator statistics would not see a hipMalloc made inside the library -- and the call can
    be recorded in a HIP graph (a capture refuses allocation) and replayed: every replay, with eager work and
    synchronisations in between and fresh query values each time, equals the workspace entry point bit for bit."""
    rng = np.random.default_rng(9)
    sc = 1.0 / math.sqrt(D)
    case = _case(tq, rng, 2, 4, 7, 3000)
    args = (case["K"], case["vp"], case["vn"], case["c"], case["vs"], D, BITS, sc)
    q = case["q"].clone()
    out = torch.empty((2, 28, D), dtype=torch.float32, device="cuda")
    tq.vonly_decode(q, *args, n_rep=7, out=out, static_scratch=True)      # first call on the device: looks the array up,
    torch.cuda.synchronize()                                              # loads the kernels' code
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(5):
        tq.vonly_decode(q, *args, n_rep=7, out=out, static_scratch=True)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, f"free device memory moved by {free_before - free_after} bytes over five calls"
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        tq.vonly_decode(q, *args, n_rep=7, out=out, static_scratch=True)
    for i in range(4):
        q.copy_(torch.from_numpy(rng.standard_normal(tuple(q.shape)).astype(np.float16)).cuda())
        out.fill_(float("nan"))
        g.replay()
        torch.cuda.synchronize()
        want = tq.vonly_decode(q, *args, n_rep=7)                         # eager, caller's workspace
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {i} differs from tq_vonly_decode_attn"


def test_static_scratch_rejects_shapes_beyond_the_array(tq):
    """More partial sums than the 4 MiB array holds: a clear error before any launch, nothing written."""
    from tqhip import _lib, ops
    lib = _lib.load()
    n_seq, n_kv, n_rep, T = 1, 4, 7, 131072           # 28 heads x 512 tiles x 130 floats = 7.5 MB
    assert lib.tq_workspace_bytes(_lib.TQ_OP_VONLY_DECODE, n_seq, n_kv * n_rep, T, D) > _lib.STATIC_SCRATCH_BYTES
    sh = ops._decode_shape(n_seq=n_seq, n_kv=n_kv, n_rep=n_rep, dim=D, bits=BITS, block_size=16, seq_len=T,
                           seq_offsets=None, k_strides=(0, T), kn_strides=(0, 0), v_strides=(0, T), vn_strides=(0, T),
                           mask=None, mask_strides=(0, 0), attn_scale=1.0, out_dtype=torch.float32)
    dummy = torch.zeros(64, dtype=torch.float32, device="cuda")       # never read: the size check comes first
    p = C.c_void_p(dummy.data_ptr())
    rc = lib.tq_vonly_decode_attn_static(p, _lib.TQ_F16, p, p, p, _lib.host_floats(o.gaussian_codebook(BITS).tolist()),
                                         p, p, C.byref(sh), C.c_void_p(0))
    assert rc == -8
    msg = lib.tq_last_error().decode()
    assert "static scratch" in msg and "tq_vonly_decode_attn" in msg
    torch.cuda.synchronize()
    assert float(dummy.abs().sum()) == 0.0
