"""numpy-facing wrapper of the CPU oracle (``liboracle.so``, built by the Makefile here).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``; the shipped library never touches it.

Every function follows the C declaration of the same name in ``oracle.h``, which cites
the reference file:line it restates.  PARITY UNPINNED (the reference leaves the point to
its compiler or to a vendor library, and holds no vector for it): the lane order of
reduce_sum in ``rms_norm_all_f16`` / ``softmax_all_f16`` (stated above those functions), and
the value stream of ``rng_fill`` against the vendor generator the reference calls (Philox
itself is pinned by the Random123 known-answer vectors).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")


def build(force: bool = False) -> str:
    """Compile liboracle.so with gcc (seconds)."""
    sources = [os.path.join(_HERE, f) for f in ("oracle.c", "oracle.h", "Makefile")]
    stale = os.path.exists(_LIB_PATH) and any(os.path.getmtime(f) > os.path.getmtime(_LIB_PATH) for f in sources if os.path.exists(f))
    if force or stale or not os.path.exists(_LIB_PATH):
        try:
            subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)
        except (OSError, subprocess.CalledProcessError):
            if force or not os.path.exists(_LIB_PATH):
                raise          # nothing usable; a merely stale library is still loaded
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        vp, i64, f32, f64, u64, sz = C.c_void_p, C.c_int64, C.c_float, C.c_double, C.c_uint64, C.c_size_t
        sigs = {
            "orc_num_threads": (C.c_int, []),
            "orc_set_num_threads": (None, [C.c_int]),
            "orc_f32_to_f16": (C.c_uint16, [f32]),
            "orc_f16_to_f32": (f32, [C.c_uint16]),
            "orc_f32_to_bf16": (C.c_uint16, [f32]),
            "orc_bf16_to_f32": (f32, [C.c_uint16]),
            "orc_e4m3fn_to_f32": (f32, [C.c_uint8]),
            "orc_f32_to_e4m3fn": (C.c_uint8, [f32]),
            "orc_e8m0_to_f32": (f32, [C.c_uint8]),
            "orc_f32_to_f16_n": (None, [vp, vp, sz]),
            "orc_f16_to_f32_n": (None, [vp, vp, sz]),
            "orc_f32_to_bf16_n": (None, [vp, vp, sz]),
            "orc_bf16_to_f32_n": (None, [vp, vp, sz]),
            "orc_fill_uniform_f32": (None, [vp, sz, u64, f32, f32]),
            "orc_fill_normal_f32": (None, [vp, sz, u64, f32, f32]),
            "orc_saxpy_f32": (None, [sz, f32, vp, vp, vp]),
            "orc_add_f32": (None, [sz, vp, vp, vp]),
            "orc_rms_norm_f16": (None, [vp, vp, vp, i64, i64, f32, i64]),
            "orc_rms_norm_f16_f64": (None, [vp, vp, vp, i64, i64, f64]),
            "orc_add_rms_norm_f16": (None, [vp, vp, vp, vp, vp, i64, i64, f32, i64]),
            "orc_qk_norm_f16": (None, [vp, vp, vp, vp, vp, i64, i64, i64, f32, i64]),
            "orc_add_f16": (None, [sz, vp, vp, vp]),
            "orc_silu_mul_f16": (None, [sz, vp, vp, vp]),
            "orc_rope_seq_f16": (None, [vp, vp, vp, i64, i64, i64, C.c_int32]),
            "orc_kv_cache_update_f16": (None, [vp, vp, vp, vp, i64, i64, i64, i64, i64]),
            "orc_fmha_decode_gqa_split": (None, [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, f32, i64]),
            "orc_attention_decode_grouped_f16": (None, [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, i64, f32, i64]),
            "orc_splitk_reduce_merge": (None, [vp, vp, vp, i64, i64, i64, i64]),
            "orc_softmax_f32": (None, [vp, vp, i64, i64, i64, i64]),
            "orc_softmax_f16": (None, [vp, vp, i64, i64, i64, i64]),
            "orc_cpu_gemm_f32": (None, [vp, vp, vp, i64, i64, i64]),
            "orc_gemm_bf16": (None, [vp, vp, vp, i64, i64, i64, vp, i64]),
            "orc_gemm_bf16_f32out": (None, [vp, vp, vp, i64, i64, i64, vp, i64]),
            "orc_fmha_ref_cpu": (None, [vp, vp, vp, vp, i64, i64, i64, i64, i64, f32, i64, i64, C.c_int, vp, i64]),
            "orc_rms_norm_f32_example": (None, [vp, vp, vp, i64, i64, f32, i64]),
            "orc_qk_norm_rope_kv_f16": (None, [vp] * 9 + [f32, i64, i64, i64, i64, i64, i64]),
            "orc_argmax_blocks_f16": (None, [vp, i64, i64, i64, vp, vp, i64]),
            "orc_lm_head_argmax_blocks_f16": (None, [vp, vp, i64, i64, i64, vp, vp, i64]),
            "orc_argmax_reduce_blocks_to_u32": (C.c_uint32, [vp, vp, i64, i64, i64]),
            "orc_attention_seq_ref": (None, [vp, vp, vp, vp, i64, i64, i64, i64, i64, f32, i64, i64, i64, C.c_int]),
            "orc_mx_quantize_e4m3": (None, [vp, vp, vp, i64, i64]),
            "orc_mx_dequantize_e4m3": (None, [vp, vp, vp, i64, i64]),
            "orc_mx_gemm_f32": (None, [vp, vp, vp, vp, vp, i64, i64, i64, f32, vp, i64]),
            "orc_e2m1_to_f32": (f32, [C.c_uint8]),
            "orc_f32_to_e2m1": (C.c_uint8, [f32]),
            "orc_nvfp4_quantize": (None, [vp, vp, vp, i64, i64]),
            "orc_nvfp4_dequantize": (None, [vp, vp, vp, i64, i64]),
            "orc_nvfp4_gemm_f32": (None, [vp, vp, vp, vp, vp, i64, i64, i64, f32, vp, i64]),
            "orc_philox4x32_10": (None, [vp, vp, vp]),
            "orc_rng_fill_f32": (None, [vp, sz, u64, u64, C.c_int, f32, f32]),
            "orc_rng_fill_f64": (None, [vp, sz, u64, u64, C.c_int, f64, f64]),
        }
        for name, (res, args) in sigs.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


def num_threads() -> int:
    return int(lib().orc_num_threads())


def set_num_threads(n: int) -> None:
    lib().orc_set_num_threads(int(n))


# ---- codecs -------------------------------------------------------------------------------
def f32_to_f16_bits(x) -> np.ndarray:
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().orc_f32_to_f16_n(_p(x), _p(out), x.size)
    return out


def f16_bits_to_f32(h) -> np.ndarray:
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().orc_f16_to_f32_n(_p(h), _p(out), h.size)
    return out


def f32_to_bf16_bits(x) -> np.ndarray:
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().orc_f32_to_bf16_n(_p(x), _p(out), x.size)
    return out


def bf16_bits_to_f32(h) -> np.ndarray:
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().orc_bf16_to_f32_n(_p(h), _p(out), h.size)
    return out


def e4m3fn_to_f32(code: int) -> float:
    return float(lib().orc_e4m3fn_to_f32(int(code)))


def f32_to_e4m3fn(v: float) -> int:
    return int(lib().orc_f32_to_e4m3fn(float(v)))


def e8m0_to_f32(code: int) -> float:
    return float(lib().orc_e8m0_to_f32(int(code)))


# ---- seeded inputs ------------------------------------------------------------------------
def uniform_f32(shape, seed: int, lo: float = -1.0, hi: float = 1.0) -> np.ndarray:
    out = np.empty(shape, np.float32)
    lib().orc_fill_uniform_f32(_p(out), out.size, seed, lo, hi)
    return out


def normal_f32(shape, seed: int, mean: float = 0.0, std: float = 1.0) -> np.ndarray:
    out = np.empty(shape, np.float32)
    lib().orc_fill_normal_f32(_p(out), out.size, seed, mean, std)
    return out


# ---- K1 -----------------------------------------------------------------------------------
def saxpy_f32(a: float, x, y) -> np.ndarray:
    x, y = _c(x, np.float32), _c(y, np.float32)
    z = np.empty_like(x)
    lib().orc_saxpy_f32(x.size, a, _p(x), _p(y), _p(z))
    return z


def add_f32(x, y) -> np.ndarray:
    x, y = _c(x, np.float32), _c(y, np.float32)
    z = np.empty_like(x)
    lib().orc_add_f32(x.size, _p(x), _p(y), _p(z))
    return z


# ---- K2 -----------------------------------------------------------------------------------
def rms_norm_f16(x_bits, w_bits, eps: float, block: int = 0) -> np.ndarray:
    x, w = _c(x_bits, np.uint16), _c(w_bits, np.uint16)
    rows, n = x.shape
    out = np.empty_like(x)
    lib().orc_rms_norm_f16(_p(x), _p(w), _p(out), rows, n, eps, block or n)
    return out


def rms_norm_f32_example(x, w, eps: float, block: int = 0) -> np.ndarray:
    """cutile-examples/examples/rms_norm.rs:17-61 (f32, square root rounded toward minus infinity)"""
    x, w = _c(x, np.float32), _c(w, np.float32)
    rows, n = x.shape
    out = np.empty_like(x)
    lib().orc_rms_norm_f32_example(_p(x), _p(w), _p(out), rows, n, eps, block)
    return out


def rms_norm_f16_f64(x_bits, w_bits, eps: float) -> np.ndarray:
    x, w = _c(x_bits, np.uint16), _c(w_bits, np.uint16)
    rows, n = x.shape
    out = np.empty_like(x)
    lib().orc_rms_norm_f16_f64(_p(x), _p(w), _p(out), rows, n, eps)
    return out


# ---- the benchmark programs' all-f16 arithmetic (numpy; every operation rounded once to f16) -------------------
# cutile-benchmarks/benches/rmsnorm.rs:20-66 and benches/softmax.rs:19-35 compute entirely in f16.  PARITY UNPINNED
# against the reference for one choice both programs leave to their compiler: the order in which reduce_sum adds the
# lanes of a tile.  The order restated here is the stride-halving tree (a[l] += a[l + step], step = L/2 .. 1).  The
# softmax's f16 exp is evaluated in f32 and rounded once.  Everything else (the per-lane accumulation over tiles, the
# scalar chain, the downward-rounded square root, the order of the two multiplications) is fixed by the programs.
# An f32 operation on two f16 values, rounded to f16, is the correctly rounded f16 operation (24 >= 2 * 11 + 2 bits),
# which is how every step below is computed.
def _h(op, a, b):
    with np.errstate(over="ignore", divide="ignore", invalid="ignore"):      # f16 overflow to inf is part of the arithmetic
        return op(a.astype(np.float32), np.asarray(b, np.float16).astype(np.float32)).astype(np.float16)


def _tree_sum_f16(a: np.ndarray) -> np.ndarray:
    """stride-halving tree over the last axis (a power of two long), one f16 rounding per addition"""
    step = a.shape[-1] // 2
    while step >= 1:
        a = _h(np.add, a[..., :step], a[..., step:2 * step])
        step //= 2
    return a[..., 0]


def sqrt_f16_toward_minus_infinity(v: np.ndarray) -> np.ndarray:
    """largest f16 whose square does not exceed v (rounding::NegativeInf): squares of f16 values are exact in f64"""
    v = np.asarray(v, np.float16)
    with np.errstate(invalid="ignore"):
        r = np.sqrt(v.astype(np.float64)).astype(np.float16)                       # nearest: at most one step above the floor
        above = np.isfinite(r) & (r.astype(np.float64) ** 2 > v.astype(np.float64))
    return np.where(above, np.nextafter(r, np.float16(-np.inf)), r).astype(np.float16)


def rms_norm_all_f16(x_bits, w_bits, eps: float, block: int) -> np.ndarray:
    """cutile-benchmarks/benches/rmsnorm.rs:20-66 -> f16 bit patterns"""
    x, w = _c(x_bits, np.uint16).view(np.float16), _c(w_bits, np.uint16).view(np.float16)
    rows, n = x.shape
    assert n % block == 0 and block & (block - 1) == 0
    acc = np.zeros((rows, block), np.float16)
    for j in range(n // block):                                  # rms = rms + tx * tx, lane by lane (:37-40)
        t = x[:, j * block:(j + 1) * block]
        acc = _h(np.add, acc, _h(np.multiply, t, t))
    total = _tree_sum_f16(acc)                                   # reduce_sum (:43)
    with np.errstate(divide="ignore", over="ignore", invalid="ignore"):
        mean = _h(np.divide, total, np.float16(n))               # rms / n (:46-48)
        inv = _h(np.divide, np.ones_like(mean), _h(np.add, mean, np.float16(eps)))
        scale = sqrt_f16_toward_minus_infinity(inv)              # :49-50
        out = _h(np.multiply, _h(np.multiply, x, scale[:, None]), w[None, :])   # tx * rms * tw (:62)
    return out.view(np.uint16)


def softmax_all_f16(x_bits, bm: int, bn: int) -> np.ndarray:
    """cutile-benchmarks/benches/softmax.rs:19-35 over [bm, bn] tiles -> f16 bit patterns; columns of a tile beyond the
    tensor read 0 and take part in max and sum"""
    x = _c(x_bits, np.uint16).view(np.float16)
    m, n = x.shape
    assert bn & (bn - 1) == 0
    tiles = -(-n // bn)
    xp = np.zeros((m, tiles * bn), np.float16)
    xp[:, :n] = x
    seg = xp.reshape(m, tiles, bn)
    mx = seg.max(axis=2, keepdims=True)
    with np.errstate(over="ignore", invalid="ignore", divide="ignore"):
        d = _h(np.subtract, seg, mx)
        num = np.exp(d.astype(np.float32)).astype(np.float16)
        den = _tree_sum_f16(num)[..., None]
        y = _h(np.divide, num, den)
    return np.ascontiguousarray(y.reshape(m, tiles * bn)[:, :n]).view(np.uint16)


# ---- transformer-block kernels ---------------------------------------------------------------
def add_rms_norm_f16(residual_bits, x_bits, w_bits, eps: float, block: int = 0):
    """-> (out, residual_out), both f16 bit patterns"""
    r, x, w = _c(residual_bits, np.uint16), _c(x_bits, np.uint16), _c(w_bits, np.uint16)
    rows, n = x.shape
    out, res = np.empty_like(x), np.empty_like(x)
    lib().orc_add_rms_norm_f16(_p(r), _p(x), _p(w), _p(out), _p(res), rows, n, eps, block or n)
    return out, res


def qk_norm_f16(q_bits, k_bits, qw_bits, kw_bits, eps: float, block: int = 0) -> np.ndarray:
    q, k = _c(q_bits, np.uint16), _c(k_bits, np.uint16)
    qw, kw = _c(qw_bits, np.uint16), _c(kw_bits, np.uint16)
    n = q.shape[1]
    out = np.empty((q.shape[0] + k.shape[0], n), np.uint16)
    lib().orc_qk_norm_f16(_p(q), _p(k), _p(qw), _p(kw), _p(out), q.shape[0], k.shape[0], n, eps, block or n)
    return out


def add_f16(lhs_bits, rhs_bits) -> np.ndarray:
    a, b = _c(lhs_bits, np.uint16), _c(rhs_bits, np.uint16)
    out = np.empty_like(a)
    lib().orc_add_f16(a.size, _p(a), _p(b), _p(out))
    return out


def silu_mul_f16(gate_bits, up_bits) -> np.ndarray:
    g, u = _c(gate_bits, np.uint16), _c(up_bits, np.uint16)
    out = np.empty_like(g)
    lib().orc_silu_mul_f16(g.size, _p(g), _p(u), _p(out))
    return out


def rope_seq_f16(x_bits, inv_freq, position_start: int) -> np.ndarray:
    x, f = _c(x_bits, np.uint16), _c(inv_freq, np.float32)
    seq, heads, d = x.shape
    assert f.size == d // 2
    out = np.empty_like(x)
    lib().orc_rope_seq_f16(_p(x), _p(f), _p(out), seq, heads, d, position_start)
    return out


def kv_cache_update_f16(new_k_bits, new_v_bits, k_cache_bits, v_cache_bits, position_start: int, seq_len: int):
    """-> (k_cache, v_cache) copies with cache[h, position_start + s] = new[s, h] for s < seq_len"""
    nk, nv = _c(new_k_bits, np.uint16), _c(new_v_bits, np.uint16)
    kc, vc = _c(k_cache_bits, np.uint16).copy(), _c(v_cache_bits, np.uint16).copy()
    heads, max_seq, d = kc.shape
    lib().orc_kv_cache_update_f16(_p(nk), _p(nv), _p(kc), _p(vc), heads, d, max_seq, position_start, seq_len)
    return kc, vc


def fmha_decode_gqa_split(q_bits, k_bits, v_bits, qk_scale: float, input_pos: int, bn: int, splits: int):
    """-> (att_partial [kv_heads, splits*group, d] f16 bits, lse_partial [kv_heads, splits*group] f32)"""
    q, k, v = _c(q_bits, np.uint16), _c(k_bits, np.uint16), _c(v_bits, np.uint16)
    kv_heads, group, d = q.shape
    max_seq = k.shape[1]
    att = np.empty((kv_heads, splits * group, d), np.uint16)
    lse = np.empty((kv_heads, splits * group), np.float32)
    lib().orc_fmha_decode_gqa_split(_p(q), _p(k), _p(v), _p(att), _p(lse), kv_heads, group, d, max_seq, bn, splits,
                                    qk_scale, input_pos)
    return att, lse


def attention_decode_grouped_f16(q_bits, k_bits, v_bits, softmax_scale: float, s_kv: int, tile_n: int, kv_len_per_split: int,
                                 splits: int):
    """experimental/attention.rs:385-846 -> (att [b, h, g, splits, d] f16 bits, lse [b, h, g, splits] f32)"""
    q, k, v = _c(q_bits, np.uint16), _c(k_bits, np.uint16), _c(v_bits, np.uint16)
    batch, heads, group, d = q.shape
    s_max = k.shape[2]
    att = np.empty((batch, heads, group, splits, d), np.uint16)
    lse = np.empty((batch, heads, group, splits), np.float32)
    lib().orc_attention_decode_grouped_f16(_p(q), _p(k), _p(v), _p(att), _p(lse), batch, heads, group, d, s_max, splits,
                                           tile_n, kv_len_per_split, softmax_scale, s_kv)
    return att, lse


def splitk_reduce_merge(att_bits, lse, group: int) -> np.ndarray:
    att, lse = _c(att_bits, np.uint16), _c(lse, np.float32)
    kv_heads, ns_group, d = att.shape
    out = np.empty((kv_heads, group, d), np.uint16)
    lib().orc_splitk_reduce_merge(_p(att), _p(lse), _p(out), kv_heads, group, d, ns_group // group)
    return out


# ---- mapped partitions ----------------------------------------------------------------------
def mapped_schedule(grid, map_shape):
    """The order in which stream items visit the tiles of a mapped partition, as a list of block-id
    tuples (one entry per partition axis, owned axes 0): item t of the stream is element t.

    cutile-compiler/src/compiler/compile_intrinsic.rs:2438-2900 states the schedule as index arithmetic
    (emit_swizzle_2d / emit_mapped_partition_schedule); here the same order is produced constructively,
    by walking it: leading streamed axes row-major; the trailing two streamed axes (m, n) in bands of
    GM tile rows, each band cut into groups of GN columns, each group column by column, rows fastest.
    A map dimension of 0 (OWNED) takes the axis out of the stream.  Pure Python: small grids only."""
    rank = len(map_shape)
    streamed = [a for a in range(rank) if map_shape[a] != 0]
    lens = [int(grid[a]) for a in streamed]
    maps = [int(map_shape[a]) for a in streamed]

    def place(coords):
        out = [0] * rank
        for a, c in zip(streamed, coords):
            out[a] = c
        return tuple(out)

    def pairs(num_m, num_n, gm, gn):
        for band in range(0, num_m, gm):
            rows = min(gm, num_m - band)
            for group in range(0, num_n, gn):
                for n in range(group, min(group + gn, num_n)):
                    for m in range(band, band + rows):
                        yield m, n

    order = []
    if len(streamed) == 1:
        order = [place((t,)) for t in range(lens[0])]
    elif len(streamed) == 2:
        gm, gn = maps
        # (1, 1) is plain row-major in the reference (tile / num_n, tile % num_n), not bands of one row
        # walked column by column -- which is the same thing: a band of one row IS a row.
        order = [place(p) for p in pairs(lens[0], lens[1], gm, gn if (gm, gn) != (1, 1) else 1)]
    elif len(streamed) == 3:
        for lead in range(lens[0]):
            order += [place((lead,) + p) for p in pairs(lens[1], lens[2], maps[1], maps[2])]
    return order


# ---- the example programs' small kernels (numpy, f32) ---------------------------------------
def relu_f32(x) -> np.ndarray:
    """cutile-examples/examples/async_mlp.rs:56-61: max_tile(0, x)"""
    x = _c(x, np.float32)
    return np.where(x > 0, x, np.float32(0)).astype(np.float32)


def dropout_f32(p: float, x_keep, n_out: int = None) -> np.ndarray:
    """cutile-examples/examples/dropout.rs:23-31: select(x_keep > p, x_keep, 0) / (1 - p), every step in f32;
    x_keep is loaded like the output tile, so positions it does not have read 0"""
    k = _c(x_keep, np.float32).reshape(-1)
    n = k.size if n_out is None else n_out
    padded = np.zeros(n, np.float32)
    padded[:min(n, k.size)] = k[:n]
    p32 = np.float32(p)
    kept = np.where(padded > p32, padded, np.float32(0)).astype(np.float32)
    return (kept / (np.float32(1) - p32)).astype(np.float32)


def scale_f32(x, scale: float) -> np.ndarray:
    """cutile-examples/examples/scale_ptr.rs:66 (tile * scale_tile), the check at :102-110"""
    return (_c(x, np.float32) * np.float32(scale)).astype(np.float32)


def matvec_f32(z, x, y, k: int = None, bk: int = 1) -> np.ndarray:
    """cutile-examples/examples/async_mlp.rs:38-54: z + x . y over k / BK whole K tiles, as cpu_gemm_f32 with one
    column (the order in which a tile's products are added is the assembler's)"""
    x, y, z = _c(x, np.float32), _c(y, np.float32), _c(z, np.float32)
    k = x.shape[1] if k is None else k
    kt = min((k // bk) * bk, x.shape[1], y.shape[0])
    return (z + cpu_gemm_f32(x[:, :kt], y[:kt].reshape(kt, 1)).reshape(-1)).astype(np.float32)


def batch_matmul_f32(a, b, k: int = None, bk: int = 1) -> np.ndarray:
    """cutile-examples/examples/batch_matmul.rs:31-43: cpu_gemm_f32 of every batch, from zero accumulators"""
    a, b = _c(a, np.float32), _c(b, np.float32)
    k = a.shape[2] if k is None else k
    kt = min((k // bk) * bk, a.shape[2], b.shape[1])
    return np.stack([cpu_gemm_f32(a[i, :, :kt], b[i, :kt, :]) for i in range(a.shape[0])])


# ---- K3 -----------------------------------------------------------------------------------
def softmax_f32(x, bm: int, bn: int) -> np.ndarray:
    x = _c(x, np.float32)
    m, n = x.shape
    y = np.zeros_like(x)
    lib().orc_softmax_f32(_p(x), _p(y), m, n, bm, bn)
    return y


def softmax_f16(x_bits, bm: int, bn: int) -> np.ndarray:
    x = _c(x_bits, np.uint16)
    m, n = x.shape
    y = np.zeros_like(x)
    lib().orc_softmax_f16(_p(x), _p(y), m, n, bm, bn)
    return y


# ---- K4 -----------------------------------------------------------------------------------
def cpu_gemm_f32(x, y) -> np.ndarray:
    x, y = _c(x, np.float32), _c(y, np.float32)
    m, k = x.shape
    k2, n = y.shape
    assert k == k2
    z = np.empty((m, n), np.float32)
    lib().orc_cpu_gemm_f32(_p(x), _p(y), _p(z), m, n, k)
    return z


def _rows_arg(rows):
    if rows is None:
        return None, None, 0
    r = _c(rows, np.int64)
    return r, _p(r), r.size


def gemm_bf16(a_bits, b_bits, rows=None, f32out: bool = False) -> np.ndarray:
    a, b = _c(a_bits, np.uint16), _c(b_bits, np.uint16)
    m, k = a.shape
    k2, n = b.shape
    assert k == k2
    keep, rp, nr = _rows_arg(rows)
    cnt = nr if rows is not None else m
    if f32out:
        c = np.empty((cnt, n), np.float32)
        lib().orc_gemm_bf16_f32out(_p(a), _p(b), _p(c), m, n, k, rp, nr)
    else:
        c = np.empty((cnt, n), np.uint16)
        lib().orc_gemm_bf16(_p(a), _p(b), _p(c), m, n, k, rp, nr)
    return c


# ---- K5 -----------------------------------------------------------------------------------
def fmha_ref_cpu(q, k, v, qk_scale: float, input_pos: int = 0, query_group_size: int = 1,
                 causal: bool = False, rows=None) -> np.ndarray:
    q, k, v = _c(q, np.float32), _c(k, np.float32), _c(v, np.float32)
    b, h, m, d = q.shape
    hkv = k.shape[1]
    keep, rp, nr = _rows_arg(rows)
    out = np.empty((nr, d) if rows is not None else (b, h, m, d), np.float32)
    lib().orc_fmha_ref_cpu(_p(q), _p(k), _p(v), _p(out), b, h, hkv, m, d, qk_scale, input_pos,
                           query_group_size, int(causal), rp, nr)
    return out


def attention_seq_ref(q, k, v, qk_scale: float, query_group_size: int, kv_len: int, query_start: int = 0,
                      causal: bool = True) -> np.ndarray:
    """q [q_len, q_heads, D], k and v [kv_heads, max_seq, D] -> out [q_len, q_heads, D] (f32)"""
    q, k, v = _c(q, np.float32), _c(k, np.float32), _c(v, np.float32)
    q_len, q_heads, d = q.shape
    kv_heads, max_seq, _ = k.shape
    assert v.shape == k.shape and kv_heads * query_group_size == q_heads
    out = np.empty((q_len, q_heads, d), np.float32)
    lib().orc_attention_seq_ref(_p(q), _p(k), _p(v), _p(out), q_len, q_heads, kv_heads, max_seq, d, qk_scale,
                                query_group_size, int(kv_len), int(query_start), int(causal))
    return out


def qk_norm_rope_kv_f16(q_bits, k_bits, v_bits, qw_bits, kw_bits, inv_freq, k_cache_bits, v_cache_bits, eps: float,
                        position_start: int):
    """fused_transformer.rs:22-345 -> (q_out bits [seq, nq, d], k_cache bits, v_cache bits); the caches are copied first"""
    q_bits, k_bits, v_bits = _c(q_bits, np.uint16), _c(k_bits, np.uint16), _c(v_bits, np.uint16)
    qw_bits, kw_bits, inv_freq = _c(qw_bits, np.uint16), _c(kw_bits, np.uint16), _c(inv_freq, np.float32)
    seq, nq, d = q_bits.shape
    nkv = k_bits.shape[1]
    kc, vc = _c(k_cache_bits, np.uint16).copy(), _c(v_cache_bits, np.uint16).copy()
    q_out = np.empty_like(q_bits)
    lib().orc_qk_norm_rope_kv_f16(_p(q_bits), _p(k_bits), _p(v_bits), _p(qw_bits), _p(kw_bits), _p(inv_freq), _p(q_out), _p(kc),
                                  _p(vc), eps, int(position_start), seq, nq, nkv, d, kc.shape[1])
    return q_out, kc, vc


# ---- KV block layout conversion (cutile-kernels/src/experimental/kvbm.rs) ----
KVBM_UNIVERSAL_TO_STACKED = {"nhd": (1, 2, 3, 0, 4), "hnd": (1, 2, 0, 3, 4)}                        # kvbm.rs:390-394
KVBM_STACKED_TO_CONTIGUOUS = {("nhd", "universal"): (3, 0, 1, 2, 4), ("hnd", "universal"): (2, 0, 1, 3, 4),
                              ("nhd", "operational_nhd"): (0, 1, 2, 3, 4), ("hnd", "operational_hnd"): (0, 1, 2, 3, 4)}   # :378-383


def kvbm_stacked_to_contiguous(stacked, stacked_layout: str, contiguous_layout: str) -> np.ndarray:
    """copy_stacked_to_contiguous_f16 (kvbm.rs:112-187).  stacked: [blocks, nl, no] + the per-(block, layer, offset) tensor
    ([nt, nh, hd] for "nhd", [nh, nt, hd] for "hnd"); returns [blocks] + the contiguous shape.  The kernel permutes every
    tile with STACKED_TO_CONTIGUOUS_MAP (:176), i.e. transposes the block by that map."""
    stacked = np.asarray(stacked)
    axes = KVBM_STACKED_TO_CONTIGUOUS[(stacked_layout, contiguous_layout)]
    return np.ascontiguousarray(np.transpose(stacked, (0,) + tuple(a + 1 for a in axes)))


def kvbm_contiguous_to_stacked(contiguous, stacked_layout: str, contiguous_layout: str) -> np.ndarray:
    """copy_contiguous_to_stacked_f16 (kvbm.rs:283-352): the inverse permutation"""
    contiguous = np.asarray(contiguous)
    axes = KVBM_STACKED_TO_CONTIGUOUS[(stacked_layout, contiguous_layout)]
    inverse = np.argsort(axes)
    return np.ascontiguousarray(np.transpose(contiguous, (0,) + tuple(int(a) + 1 for a in inverse)))


# ---- greedy sampling and row gathers (cutile-kernels/src/argmax.rs, embeddings.rs, pointwise.rs) ----
def argmax_blocks_f16(logits_bits, block_size: int, length: int, num_blocks: int = None):
    """-> (block_max f32 [blocks], block_idx u32 [blocks])"""
    logits_bits = _c(logits_bits, np.uint16)
    n = logits_bits.shape[0]
    nb = num_blocks if num_blocks is not None else -(-n // block_size)
    bm, bi = np.empty(nb, np.float32), np.empty(nb, np.uint32)
    lib().orc_argmax_blocks_f16(_p(logits_bits), n, block_size, length, _p(bm), _p(bi), nb)
    return bm, bi


def lm_head_argmax_blocks_f16(weight_bits, hidden_bits, vocab_size: int, num_blocks: int = None):
    weight_bits, hidden_bits = _c(weight_bits, np.uint16), _c(hidden_bits, np.uint16)
    rows, k = weight_bits.shape
    assert hidden_bits.size == k
    nb = num_blocks if num_blocks is not None else -(-rows // 64)
    bm, bi = np.empty(nb, np.float32), np.empty(nb, np.uint32)
    lib().orc_lm_head_argmax_blocks_f16(_p(weight_bits), _p(hidden_bits), rows, k, vocab_size, _p(bm), _p(bi), nb)
    return bm, bi


def argmax_reduce_blocks_to_u32(block_max, block_idx, num_blocks: int, block_size: int = None) -> int:
    block_max, block_idx = _c(block_max, np.float32), _c(block_idx, np.uint32)
    n = block_max.shape[0]
    bs = block_size if block_size is not None else max(256, -(-num_blocks // 256) * 256)
    return int(lib().orc_argmax_reduce_blocks_to_u32(_p(block_max), _p(block_idx), n, bs, num_blocks))


def embedding_batch_f16(token_ids, table_bits) -> np.ndarray:
    """embeddings.rs:21-41: out[r, :] = table[token_ids[r], :], zeros for a token beyond the table (padded tile load)"""
    token_ids, table_bits = np.asarray(token_ids, np.int64), _c(table_bits, np.uint16)
    out = np.zeros((token_ids.shape[0], table_bits.shape[1]), np.uint16)
    ok = (token_ids >= 0) & (token_ids < table_bits.shape[0])
    out[ok] = table_bits[token_ids[ok]]
    return out


def gather_row_f16(src_bits, row_idx: int, width: int = None) -> np.ndarray:
    """pointwise.rs:86-99: out[c] = src[row_idx, c], zeros where src has no such element"""
    src_bits = _c(src_bits, np.uint16)
    width = src_bits.shape[1] if width is None else width
    out = np.zeros(width, np.uint16)
    if 0 <= row_idx < src_bits.shape[0]:
        m = min(width, src_bits.shape[1])
        out[:m] = src_bits[row_idx, :m]
    return out


# ---- K6 -----------------------------------------------------------------------------------
def mx_quantize_e4m3(src):
    src = _c(src, np.float32)
    rows, k = src.shape
    assert k % 32 == 0
    data = np.empty((rows, k), np.uint8)
    scales = np.empty((rows, k // 32), np.uint8)
    lib().orc_mx_quantize_e4m3(_p(src), _p(data), _p(scales), rows, k)
    return data, scales


def mx_dequantize_e4m3(data, scales) -> np.ndarray:
    data, scales = _c(data, np.uint8), _c(scales, np.uint8)
    rows, k = data.shape
    dst = np.empty((rows, k), np.float32)
    lib().orc_mx_dequantize_e4m3(_p(data), _p(scales), _p(dst), rows, k)
    return dst


def mx_gemm_f32(x, y, xs, ys, alpha: float = 1.0, rows=None) -> np.ndarray:
    x, y, xs, ys = _c(x, np.uint8), _c(y, np.uint8), _c(xs, np.uint8), _c(ys, np.uint8)
    m, k = x.shape
    n, k2 = y.shape
    assert k == k2
    keep, rp, nr = _rows_arg(rows)
    z = np.empty((nr if rows is not None else m, n), np.float32)
    lib().orc_mx_gemm_f32(_p(x), _p(y), _p(xs), _p(ys), _p(z), m, n, k, alpha, rp, nr)
    return z


# ---- NVFP4 ----------------------------------------------------------------------------------
def e2m1_to_f32(nibble: int) -> float:
    return float(lib().orc_e2m1_to_f32(nibble))


def f32_to_e2m1(v: float) -> int:
    return int(lib().orc_f32_to_e2m1(v))


def nvfp4_quantize(src):
    """-> (packed e2m1 pairs [rows, k/2] uint8, e4m3fn scales [rows, k/16] uint8)"""
    src = _c(src, np.float32)
    rows, k = src.shape
    assert k % 16 == 0
    data = np.empty((rows, k // 2), np.uint8)
    scales = np.empty((rows, k // 16), np.uint8)
    lib().orc_nvfp4_quantize(_p(src), _p(data), _p(scales), rows, k)
    return data, scales


def nvfp4_dequantize(data, scales) -> np.ndarray:
    data, scales = _c(data, np.uint8), _c(scales, np.uint8)
    rows, kp = data.shape
    dst = np.empty((rows, kp * 2), np.float32)
    lib().orc_nvfp4_dequantize(_p(data), _p(scales), _p(dst), rows, kp * 2)
    return dst


def nvfp4_gemm_f32(x, y, xs, ys, alpha: float = 1.0, rows=None) -> np.ndarray:
    x, y, xs, ys = _c(x, np.uint8), _c(y, np.uint8), _c(xs, np.uint8), _c(ys, np.uint8)
    m, kp = x.shape
    n, kp2 = y.shape
    assert kp == kp2
    keep, rp, nr = _rows_arg(rows)
    z = np.empty((nr if rows is not None else m, n), np.float32)
    lib().orc_nvfp4_gemm_f32(_p(x), _p(y), _p(xs), _p(ys), _p(z), m, n, kp * 2, alpha, rp, nr)
    return z


def philox4x32_10(counter, key) -> np.ndarray:
    """one Philox4x32-10 block: counter 4 x u32, key 2 x u32 -> 4 x u32"""
    c, k = _c(counter, np.uint32), _c(key, np.uint32)
    out = np.empty(4, np.uint32)
    lib().orc_philox4x32_10(_p(c), _p(k), _p(out))
    return out


def rng_fill(n: int, seed: int, offset: int = 0, kind: str = "uniform", mean: float = 0.0, std: float = 1.0, dtype=np.float32) -> np.ndarray:
    """what cutile_rng_{uniform,normal}_{f32,f64} write for (seed, stream offset in Philox blocks)"""
    out = np.empty(n, dtype)
    fn = lib().orc_rng_fill_f32 if dtype == np.float32 else lib().orc_rng_fill_f64
    fn(_p(out), n, seed, offset, 0 if kind == "uniform" else 1, mean, std)
    return out
