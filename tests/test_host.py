"""CPU-side tests: the C-ABI library loads and exports every declared symbol, argument errors are
raised before any launch, and the host logic (sign generator, tables, packing, meta strings,
masks) matches the oracle.  No kernel is launched here."""
import ctypes
import os
import re

import numpy as np
import pytest

torch = pytest.importorskip("torch")

import tqhip  # noqa: E402
from tqhip import _lib, ops  # noqa: E402
from oracle import polarquant_oracle as o  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    header = open(os.path.join(ROOT, "include", "tqhip.h")).read()
    declared = set(re.findall(r"\b(tq_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations parsed"
    assert declared == set(_lib.PROTOTYPES), declared ^ set(_lib.PROTOTYPES)
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.tq_version() >= 100
    assert lib.tq_status_string(-3) == b"bad bits"


def test_decode_shape_struct_matches_header_size():
    # 6 int32 + int64 + ptr + 8 int64 + ptr + 2 int64 + float + 2 int32 (+ 4 bytes tail padding)
    assert ctypes.sizeof(_lib.DecodeShape) == 6 * 4 + 8 + 8 + 8 * 8 + 8 + 2 * 8 + 4 + 4 + 4 + 4


def test_struct_mirrors_match_the_header_as_a_c_compiler_lays_it_out(tmp_path):
    """include/tqhip.h is plain C: gcc compiles a probe that prints size and field offsets of every struct
    the binding mirrors, and the ctypes mirrors must agree field by field."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no C compiler")
    mirrors = {"tq_decode_shape": _lib.DecodeShape, "tq_vonly_cache_desc": _lib.VOnlyCacheDesc,
               "tq_packed_cache_desc": _lib.PackedCacheDesc}
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "tqhip.h"', 'int main(void) {']
    for cname, mirror in mirrors.items():
        lines.append(f'  printf("{cname} size %zu\\n", sizeof({cname}));')
        for fname, _ in mirror._fields_:
            lines.append(f'  printf("{cname} {fname} %zu\\n", offsetof({cname}, {fname}));')
    lines += ['  return 0;', '}']
    src = tmp_path / "abi_probe.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "abi_probe"
    inc = os.path.join(ROOT, "include")
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", inc, str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    seen = 0
    for line in out.splitlines():
        cname, fname, value = line.split()
        mirror = mirrors[cname]
        want = ctypes.sizeof(mirror) if fname == "size" else getattr(mirror, fname).offset
        assert int(value) == want, (cname, fname, value, want)
        seen += 1
    assert seen == sum(len(m._fields_) + 1 for m in mirrors.values())


def test_argument_errors_without_launch():
    lib = _lib.load()
    null = ctypes.c_void_p(0)
    b = _lib.host_floats([0.0] * 7)
    assert lib.tq_encode(null, 1, null, b, null, null, 1, 4, 0, 0, 128, 5, 0, null) == -3
    assert b"Unsupported bit width: 5" in lib.tq_last_error()
    assert lib.tq_encode(null, 1, null, b, null, null, 1, 4, 0, 0, 96, 3, 0, null) == -2
    assert b"power of 2" in lib.tq_last_error()
    assert lib.tq_encode(null, 7, null, b, null, null, 1, 4, 0, 0, 128, 3, 0, null) == -6
    assert lib.tq_encode(null, 1, null, b, null, null, 1, 4, 0, 0, 128, 3, 0, null) == -1
    assert lib.tq_encode(null, 1, null, b, null, null, 0, 4, 0, 0, 128, 3, 0, null) == 0   # empty: no-op
    assert lib.tq_prerot_qk_scores(null, null, null, b, null, 4, 0, 16, 0, 0, 128, 3, 0, null) == -4
    assert lib.tq_sparse_v_matvec(null, null, null, b, null, null, null, 0, 4, 7, 16, 0, 0, 512, 3, 0.0, 0, null) == -2
    assert b"dim > 256" in lib.tq_last_error()
    sh = _lib.DecodeShape()
    sh.n_seq, sh.n_kv_heads, sh.n_rep, sh.dim, sh.bits, sh.block_size, sh.seq_len = 1, 2, 1, 128, 3, 33, 8
    rc = lib.tq_flash_decode(null, null, null, null, null, b, b, null, null, null, 0, ctypes.byref(sh), null)
    assert rc == -7 and b"block_size must be in 1..32" in lib.tq_last_error()
    with pytest.raises(ValueError, match="block_size must be in 1..32"):
        _lib.check(rc)
    sh.block_size, sh.dim = 16, 256
    assert lib.tq_flash_decode(null, null, null, null, null, b, b, null, null, null, 0, ctypes.byref(sh), null) == -2
    with pytest.raises(RuntimeError):
        _lib.check(-8)
    assert lib.tq_workspace_bytes(0, 1, 28, 32768, 128) == 28 * 128 * 130 * 4
    assert lib.tq_workspace_bytes(2, 1, 28, 32768, 128) == 28 * 128 * 130 * 4
    # the single-call decode steps validate descriptor, position and pointers before any launch
    for name, desc_t in (("tq_vonly_decode_step", _lib.VOnlyCacheDesc), ("tq_packed_decode_step", _lib.PackedCacheDesc)):
        fn, fn_at = getattr(lib, name), getattr(lib, name + "_at")
        assert fn(None, null, 1, null, 1, null, 1, null, 1, 0, 0.1, null) == -1
        assert fn_at(None, null, 1, null, 1, null, 1, null, 1, null, 0.1, null) == -1
        d = desc_t()
        d.n_seq, d.n_kv_heads, d.n_rep, d.dim, d.bits, d.t_alloc = 1, 4, 7, 128, 3, 256
        assert fn(ctypes.byref(d), null, 1, null, 1, null, 1, null, 1, 256, 0.1, null) == -9
        assert b"outside the storage" in lib.tq_last_error()
        assert fn(ctypes.byref(d), null, 1, null, 1, null, 1, null, 1, 5, 0.1, null) == -1     # null storage
        assert fn_at(ctypes.byref(d), null, 1, null, 1, null, 1, null, 1, null, 0.1, null) == -1
        d.bits = 5
        assert fn(ctypes.byref(d), null, 1, null, 1, null, 1, null, 1, 5, 0.1, null) == -3
    assert lib.tq_vonly_append(null, 1, null, 9, null, b, null, null, null, null, 1, 1, 0, 0, 0, 0, 128, 3, 0, null) == -6
    assert lib.tq_vonly_append(null, 1, null, 1, null, b, null, null, null, null, 0, 1, 0, 0, 0, 0, 128, 3, 0, null) == 0
    assert lib.tq_vonly_append_at(null, 1, null, 1, null, b, null, null, null, null, 1, 1, 8, 128, 3, 0, null, null) == -1


def test_kernels_refuse_cpu_tensors():
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        tqhip.fused_quantize(torch.zeros(2, 128), torch.ones(128), [0.0] * 7, 128, 3)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        tqhip.prerotate_query(torch.zeros(2, 128), torch.ones(128))
    with pytest.raises(ValueError, match="expects"):
        tqhip.prerotate_query(torch.zeros(128), torch.ones(128))
    with pytest.raises(KeyError):
        tqhip.fused_quantize(torch.zeros(2, 128), torch.ones(128), [0.0], 128, 5)
    with pytest.raises(ValueError, match="power of 2"):
        tqhip.sparse_v_matvec(torch.zeros(2, 4), torch.zeros(2, 4, 13), torch.zeros(2, 4), [0.0] * 8,
                              torch.ones(96), 96, 3)


def test_mlx_sign_stream_hash_known_answers_and_restatements_agree():
    """Threefry-2x32-20 against the Random123 known-answer vectors (zero, all-ones, digits of pi), in the package's
    scalar form and the oracle's vectorised one; the two restatements of MLX's sign stream (rotation.py:47-49) agree
    for even and odd d and seeds above 2^32; the default generator is unchanged.  The word layout of that stream is
    not pinned by anything available offline."""
    from tqhip.rotation import mlx_sign_pattern, threefry2x32
    kats = (((0, 0), (0, 0), (0x6B200159, 0x99BA4EFE)),
            ((0xFFFFFFFF, 0xFFFFFFFF), (0xFFFFFFFF, 0xFFFFFFFF), (0x1CB996FC, 0xBB002BE7)),
            ((0x13198A2E, 0x03707344), (0x243F6A88, 0x85A308D3), (0xC4923A9C, 0x483DF7A0)))
    for key, count, want in kats:
        assert threefry2x32(key, count) == want
        a, b = o.threefry2x32(key[0], key[1], [count[0]], [count[1]])
        assert (int(a[0]), int(b[0])) == want
    for d, seed in ((128, 42), (128, 43), (64, 7), (256, 0), (33, 5), (128, (3 << 32) + 9)):
        got = tqhip.random_diagonal_sign(d, seed, stream="mlx").numpy()
        assert np.array_equal(got, o.mlx_random_diagonal_sign(d, seed))
        assert got.dtype == np.float32 and set(np.unique(got)) <= {-1.0, 1.0}
        assert mlx_sign_pattern(d, seed) == got.tolist()
    assert abs(float(tqhip.random_diagonal_sign(4096, 1, stream="mlx").mean())) < 0.08
    assert not np.array_equal(tqhip.random_diagonal_sign(128, 42, stream="mlx").numpy(), tqhip.random_diagonal_sign(128, 42).numpy())
    with pytest.raises(ValueError, match="stream"):
        tqhip.random_diagonal_sign(128, 42, stream="jax")


def test_sign_generator_and_tables_match_oracle():
    for d, seed in ((128, 42), (128, 43), (64, 7), (256, 0)):
        assert np.array_equal(tqhip.random_diagonal_sign(d, seed).numpy(), o.random_diagonal_sign(d, seed))
    from tqhip.quantizer import gaussian_boundaries, gaussian_codebook
    for bits in (1, 2, 3, 4):
        c = gaussian_codebook(bits)
        assert np.array_equal(c.numpy(), o.gaussian_codebook(bits))
        assert np.array_equal(gaussian_boundaries(c).numpy(), o.gaussian_boundaries(o.gaussian_codebook(bits)))
    with pytest.raises(ValueError, match="Unsupported bit width"):
        gaussian_codebook(5)


@pytest.mark.parametrize("bits,dim", [(1, 128), (2, 32), (3, 128), (3, 64), (4, 64)])
def test_pack_unpack_match_oracle(bits, dim):
    rng = np.random.default_rng(bits)
    idx = rng.integers(0, 2 ** bits, size=(3, 7, dim)).astype(np.uint8)
    p = tqhip.pack_indices(torch.from_numpy(idx), bits)
    assert p.dtype == torch.uint32 and p.shape == (3, 7, tqhip.packed_dim(dim, bits))
    assert np.array_equal(p.numpy(), o.pack_indices(idx, bits))
    assert np.array_equal(tqhip.unpack_indices(p, bits, dim).numpy(), idx)
    assert tqhip.packed_dim(128, 3) == 13


def test_cache_meta_state_and_masks_on_host():
    c = tqhip.TurboQuantKVCache(bits=3, seed=9)
    assert c.meta_state == "0,3,9,0,0,float16" and c.state == [] and c.empty() and c.nbytes == 0
    assert c.compression_ratio == 1.0
    c.meta_state = "12,4,5,64,128,bfloat16"
    assert (c.offset, c.quant_bits, c.seed, c._k_dim, c._v_dim, c._dtype) == (12, 4, 5, 64, 128, torch.bfloat16)
    c.meta_state = "3,2,1,0,128"
    assert c._k_dim is None and c._dtype == torch.float16
    v = tqhip.VOnlyTurboQuantCache(bits=2, seed=11)
    assert v.meta_state == "VOnlyTQ,2,11,0,2,11,0,0,float16" and v.empty() and v.state == []
    m = tqhip.create_causal_mask(3, offset=2)
    assert m.tolist() == [[True, True, True, False, False], [True] * 4 + [False], [True] * 5]
    kv = tqhip.KVCache()
    k = torch.randn(1, 2, 300, 16)
    ko, vo = kv.update_and_fetch(k, k)
    assert kv.keys.shape[2] == 512 and kv.offset == 300 and torch.equal(ko, k)
    kv.update_and_fetch(k[..., :5, :], k[..., :5, :])
    assert kv.offset == 305 and kv.trim(10) == 10 and kv.size() == 295
    assert kv.make_mask(1) is None and kv.make_mask(2) == "causal"
    r = tqhip.KVCache.from_state(kv.state)
    assert r.offset == 295 and torch.equal(r.keys, k[..., :295, :])


def test_patch_install_and_restore_on_host():
    """patch.py:44-90: apply_patch replaces the attribute on every module given, once; remove_patch
    puts back what was there (or removes the attribute when there was none)."""
    import types
    import tqhip
    from tqhip import patch
    a = types.SimpleNamespace(scaled_dot_product_attention=len)
    b = types.SimpleNamespace()
    tqhip.apply_patch(a, b)
    tqhip.apply_patch(a)
    assert a.scaled_dot_product_attention is patch.scaled_dot_product_attention
    assert b.scaled_dot_product_attention is patch.scaled_dot_product_attention
    tqhip.remove_patch()
    assert a.scaled_dot_product_attention is len and not hasattr(b, "scaled_dot_product_attention")
    tqhip.remove_patch()                                   # nothing left to undo


def test_offsets_check_on_host():
    """The ragged wrappers' offsets check: dtype, count and layout always; order and range with validate=True."""
    good = torch.tensor([0, 5, 9], dtype=torch.int32)
    rows = torch.zeros((2, 9, 13), dtype=torch.int32)
    ops._check_offsets(good, 2, True, k_packed=rows)
    with pytest.raises(ValueError, match="int32"):
        ops._check_offsets(torch.cumsum(torch.tensor([0, 5, 4]), 0), 2, False)
    with pytest.raises(ValueError, match="n_seq"):
        ops._check_offsets(good, 3, False)
    with pytest.raises(ValueError, match="int32"):
        ops._check_offsets(torch.tensor([0, 1, 5, 2, 9], dtype=torch.int32)[::2], 2, False)      # not contiguous
    with pytest.raises(ValueError, match="never decrease"):
        ops._check_offsets(torch.tensor([0, 7, 5], dtype=torch.int32), 2, True)
    with pytest.raises(ValueError, match="never decrease"):
        ops._check_offsets(torch.tensor([-1, 2, 5], dtype=torch.int32), 2, True)
    with pytest.raises(ValueError, match="holds 9"):
        ops._check_offsets(torch.tensor([0, 5, 10], dtype=torch.int32), 2, True, k_packed=rows)
    ops._check_offsets(torch.tensor([0, 5, 10], dtype=torch.int32), 2, False, k_packed=rows)      # unchecked by default


def test_explicit_sign_vectors_are_validated_on_host():
    from tqhip.cache import _Quantizer, _checked_signs
    s = np.where(np.arange(128) % 3 == 0, -1.0, 1.0).astype(np.float32)
    q = _Quantizer(128, 3, seed=42, device="cpu", signs=s)
    assert q.signs.dtype == torch.float32 and np.array_equal(q.signs.numpy(), s)
    assert not np.array_equal(_Quantizer(128, 3, seed=42, device="cpu").signs.numpy(), s)
    assert np.array_equal(_checked_signs(torch.from_numpy(s).double(), 128, "cpu").numpy(), s)    # any float dtype
    for bad in (np.ones(64, np.float32), np.zeros(128, np.float32), np.ones((2, 64), np.float32), 0.5 * s):
        with pytest.raises(ValueError):
            _checked_signs(bad, 128, "cpu")
    c = tqhip.TurboQuantKVCache(bits=3, k_signs=s, v_signs=-s)
    c._ensure_quantizer(128, 128, torch.device("cpu"))
    assert np.array_equal(c._k_q.signs.numpy(), s) and np.array_equal(c._v_q.signs.numpy(), -s)
    v = tqhip.VOnlyTurboQuantCache(bits=3, v_signs=s)
    v._v_tq._ensure_quantizer(128, 128, torch.device("cpu"))
    assert np.array_equal(v._v_tq._v_q.signs.numpy(), s)


def test_sign_stream_argument_selects_the_generator_on_host():
    """sign_stream='mlx' on the constructors and on from_state expands the seed (and seed + 1 for the values)
    by the restated MLX stream; 'native' (default) by this package's; explicit vectors win; bad names raise."""
    dev = torch.device("cpu")
    mlx_k = tqhip.random_diagonal_sign(128, 7, stream="mlx").numpy()
    mlx_v = tqhip.random_diagonal_sign(128, 8, stream="mlx").numpy()
    nat_k = tqhip.random_diagonal_sign(128, 7).numpy()
    c = tqhip.TurboQuantKVCache(bits=3, seed=7, sign_stream="mlx")
    c._ensure_quantizer(128, 128, dev)
    assert np.array_equal(c._k_q.signs.numpy(), mlx_k) and np.array_equal(c._v_q.signs.numpy(), mlx_v)
    d = tqhip.TurboQuantKVCache(bits=3, seed=7)
    d._ensure_quantizer(128, 128, dev)
    assert d.sign_stream == "native" and np.array_equal(d._k_q.signs.numpy(), nat_k)
    e = tqhip.TurboQuantKVCache(bits=3, seed=7, sign_stream="mlx", k_signs=nat_k)
    e._ensure_quantizer(128, 128, dev)
    assert np.array_equal(e._k_q.signs.numpy(), nat_k) and np.array_equal(e._v_q.signs.numpy(), mlx_v)
    v = tqhip.VOnlyTurboQuantCache(bits=3, seed=7, sign_stream="mlx")
    v._v_tq._ensure_quantizer(128, 128, dev)
    assert np.array_equal(v._v_tq._v_q.signs.numpy(), mlx_v)
    # an empty serialised cache restores on the host: the stream choice survives until the first insert
    meta = "0,3,7,0,0,float16"                                # dims unknown: no quantiser (and no device) yet
    r = tqhip.TurboQuantKVCache.from_state([], meta, sign_stream="mlx")
    assert r.sign_stream == "mlx" and r.seed == 7
    r._ensure_quantizer(128, 128, dev)
    assert np.array_equal(r._k_q.signs.numpy(), mlx_k)
    rv = tqhip.VOnlyTurboQuantCache.from_state([], f"VOnlyTQ,3,7,{meta}", sign_stream="mlx")
    rv._v_tq._ensure_quantizer(128, 128, dev)
    assert np.array_equal(rv._v_tq._v_q.signs.numpy(), mlx_v)
    for make in (lambda: tqhip.TurboQuantKVCache(sign_stream="numpy"),
                 lambda: tqhip.VOnlyTurboQuantCache(sign_stream=""),
                 lambda: tqhip.TurboQuantKVCache.from_state([], meta, sign_stream="MLX"),
                 lambda: tqhip.VOnlyTurboQuantCache.from_state([], f"VOnlyTQ,3,7,{meta}", sign_stream=None)):
        with pytest.raises(ValueError, match="sign_stream"):
            make()


@pytest.mark.parametrize("have_k,have_v,offset,extra", [(1024, 1024, 1000, 2000), (1512, 1536, 1500, 1),
                                                         (300, 300, 300, 1), (556, 512, 301, 1), (0, 0, 0, 5)])
def test_vonly_cache_brings_keys_and_values_to_one_capacity(have_k, have_v, offset, extra):
    """The capacity rule of the V-only cache on host tensors (no kernel involved): whatever capacities the key
    cache and the packed values have drifted to (1000-token prompt; 1000 + 500 chunks; from_state slices; from_state
    then one insert through the two storages' own growth rules), reserve() leaves both contiguous with ONE capacity,
    a multiple of 256 with room for the request, and the first `offset` positions unchanged."""
    B, H, D = 1, 2, 128
    c = tqhip.VOnlyTurboQuantCache(bits=3)
    kc, tq = c._k_cache, c._v_tq
    g = torch.Generator().manual_seed(have_k + offset)
    if have_k:
        kc.keys = torch.randn((B, H, have_k + 3, D), generator=g).to(torch.float16)[:, :, :have_k]     # a slice, not contiguous
        kc.values = torch.randn((B, H, have_k + 3, D), generator=g).to(torch.float16)[:, :, :have_k]
        tq.v_packed = torch.randint(0, 2 ** 30, (B, H, have_v + 5, 13), generator=g, dtype=torch.int32)[:, :, :have_v].view(torch.uint32)
        tq.v_norms = torch.rand((B, H, have_v + 5), generator=g)[:, :, :have_v]
        tq._v_pdim, tq._v_dim = 13, D
    kc.offset = tq.offset = offset
    before = [t[..., :offset, :].clone() if t.dim() == 4 else t[..., :offset].clone()
              for t in (kc.keys, kc.values, tq.v_packed, tq.v_norms)] if have_k else None
    c.reserve(B, H, extra, D, device="cpu")
    n = kc.keys.shape[2]
    assert n == tq.v_packed.shape[2] == tq.v_norms.shape[2] == kc.values.shape[2]
    assert n % 256 == 0 and n >= offset + extra and n >= max(have_k, have_v)
    assert all(t.is_contiguous() for t in (kc.keys, kc.values, tq.v_packed, tq.v_norms))
    if before:
        after = [kc.keys[..., :offset, :], kc.values[..., :offset, :], tq.v_packed[..., :offset, :], tq.v_norms[..., :offset]]
        for x, y in zip(before, after):
            assert torch.equal(x.view(torch.int32) if x.dtype == torch.uint32 else x, y.view(torch.int32) if y.dtype == torch.uint32 else y)
    addr = kc.keys.data_ptr()
    c.reserve(B, H, extra, D, device="cpu")                  # nothing moves when both agree and have room
    assert kc.keys.data_ptr() == addr
    c.set_offset(n)
    with pytest.raises(ValueError):
        c.set_offset(n + 1)


def test_matrix_core_shape_predicates():
    """The one-call steps (packed or fp16 keys) cover d = 128 at every width the reference's caches accept
    (cache.py:60, v_only_cache.py:41, adaptive.py:26)."""
    for bits in (1, 2, 3, 4):
        assert ops.vonly_threshold_supported(128, bits, 7)
        assert ops.vonly_sparse_supported(128, bits, 7)
    for dim, bits, n_rep in ((64, 3, 1), (256, 3, 4), (128, 3, 17), (128, 3, 0), (128, 5, 1), (128, 0, 1)):
        assert not ops.vonly_threshold_supported(dim, bits, n_rep)
        assert not ops.vonly_sparse_supported(dim, bits, n_rep)


def _plan_restated(n_seq, n_kv, max_len, ragged, masked):
    """The step rule of the streaming flash pass, restated: steps of 256 positions per workgroup, 0 for the tile pass."""
    if masked:
        return 0
    steps, groups = -(-max_len // 256), n_seq * n_kv
    if groups * steps <= 512:
        return 0
    cap = 4 if ragged else 8
    wgs = lambda n: groups * -(-steps // n)
    alone = next((n for n in range(2, cap + 1) if wgs(n) <= 256), 0)
    shared = next((n for n in range(2, cap + 1) if wgs(n) <= 512), 0)
    if shared:
        return alone if alone and alone * 27 <= shared * 42 else shared
    best, best_n = None, cap
    for n in range(2, cap + 1):
        rest = wgs(n) % 512
        cost = (wgs(n) // 512) * (42 * n + 50) + (0 if rest == 0 else (27 if rest <= 256 else 42) * n + 50)
        if best is None or cost <= best:
            best, best_n = cost, n
    return best_n


def test_flash_decode_plan_follows_its_rule_on_host():
    """tq_flash_decode_plan is host arithmetic (no launch): known picks, and a grid of shapes against the restated rule.
    Every pick leaves no workgroup without work at the front of a sequence: steps * 256 * (workgroups - 1) < length."""
    lib = _lib.load()
    plan = lambda *a: lib.tq_flash_decode_plan(*a)
    assert plan(1, 4, 4096, 0, 0) == 0                      # short: the tile pass
    assert plan(16, 8, 32768, 1, 1) == 0                    # masked: the tile pass
    assert plan(1, 8, 16384, 0, 0) == 0                     # exactly 512 steps: one eight-wave tile per CU
    assert plan(1, 8, 18432, 0, 0) == 3                     # one four-wave workgroup per CU (192) beats two (288)
    assert plan(1, 8, 32768, 0, 0) == 2
    assert plan(1, 8, 131072, 0, 0) == 8
    assert plan(16, 8, 32768, 1, 0) == 4                    # ragged batches stop at four steps
    assert plan(16, 8, 10240, 0, 0) == 5                    # whole rounds: 1024 workgroups of five steps, not 640 of eight
    for n_seq in (1, 2, 3, 5, 16):
        for n_kv in (1, 4, 8):
            for max_len in (1, 255, 256, 4097, 16384, 16385, 20000, 36864, 65536, 131072, 1000000):
                for ragged in (0, 1):
                    for masked in (0, 1):
                        got = plan(n_seq, n_kv, max_len, ragged, masked)
                        assert got == _plan_restated(n_seq, n_kv, max_len, ragged, masked), (n_seq, n_kv, max_len, ragged, masked)
                        if got:
                            assert 2 <= got <= (4 if ragged else 8)
                            assert got * 256 * (-(-max_len // (got * 256)) - 1) < max_len
