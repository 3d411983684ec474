"""numpy/ctypes binding of oracle/liboracle.so (the CPU restatement in moe_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the cpu_baseline
leg of bench.py, as the checker and the timed CPU baseline.  The GPU package never imports it.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liboracle.so")

_c = ctypes
_vp, _i, _ll, _f, _u = _c.c_void_p, _c.c_int, _c.c_longlong, _c.c_float, _c.c_uint


def build(force=False):
    """Compile liboracle.so with the Makefile next to this file."""
    src = os.path.join(_HERE, "moe_oracle.c")
    if force or not os.path.exists(LIB_PATH) or os.path.getmtime(LIB_PATH) < os.path.getmtime(src):
        if force and os.path.exists(LIB_PATH):
            os.remove(LIB_PATH)
        subprocess.run(["make", "-C", _HERE, "liboracle.so"], check=True, capture_output=True)
    return LIB_PATH


def _load():
    build()  # compiles when the library is missing or older than its source
    lib = ctypes.CDLL(LIB_PATH)
    sig = {
        "oracle_max_threads": (_i, []),
        "oracle_matmul": (None, [_vp, _vp, _vp, _i, _i]),
        "oracle_rmsnorm": (None, [_vp, _vp, _vp, _i]),
        "oracle_softmax": (None, [_vp, _i]),
        "oracle_topk": (_i, [_vp, _vp, _vp, _i, _i]),
        "oracle_topk_qsort": (_i, [_vp, _vp, _vp, _i, _i]),
        "oracle_swiglu": (None, [_vp, _vp, _i, _f]),
        "oracle_moe_block": (_i, [_i, _i, _i, _i, _i, _f] + [_vp] * 11),
        "oracle_moe_layer": (_i, [_i, _i, _i, _i, _i, _f] + [_vp] * 12),
        "oracle_mxfp4_to_bf16_bits": (_c.c_uint16, [_u, _u]),
        "oracle_dequant_mxfp4": (None, [_vp, _vp, _ll, _vp]),
        "oracle_dequant_mxfp4_f32": (None, [_vp, _vp, _ll, _vp]),
        "oracle_bf16_to_f32": (None, [_vp, _ll, _vp]),
        "oracle_f32_to_bf16": (None, [_vp, _ll, _vp]),
        "oracle_bucket": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp, _vp, _vp]),
        "oracle_classify_queues": (None, [_vp, _i, _i, _f, _f, _vp, _vp, _vp]),
        "oracle_synth_normal_table": (None, [_vp]),
        "oracle_synth_normal_f32": (None, [_vp, _ll, _vp, _f, _u, _u, _ll]),
        "oracle_synth_normal_bf16": (None, [_vp, _ll, _vp, _f, _u, _u, _ll]),
        "oracle_synth_bytes": (None, [_vp, _ll, _u, _u, _ll]),
        "oracle_synth_range_bytes": (None, [_vp, _ll, _u, _u, _u, _u, _ll]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    return lib


_lib = _load()


def _p(a):
    return None if a is None else a.ctypes.data_as(_vp)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def max_threads():
    return _lib.oracle_max_threads()


def matmul(x, w):
    """w [d,n] @ x [n] with float products and double accumulation (src/run.cpp:341-354)."""
    x, w = _f32(x), _f32(w)
    d, n = w.shape
    out = np.empty(d, dtype=np.float32)
    _lib.oracle_matmul(_p(out), _p(x), _p(w), n, d)
    return out


def rmsnorm(x, weight):
    x, weight = _f32(x), _f32(weight)
    out = np.empty_like(x)
    _lib.oracle_rmsnorm(_p(out), _p(x), _p(weight), x.shape[-1])
    return out


def softmax(x):
    x = _f32(x).copy()
    _lib.oracle_softmax(_p(x), x.shape[-1])
    return x


def topk(score, k, use_qsort=False):
    score = _f32(score)
    v = np.empty(k, dtype=np.float32)
    i = np.empty(k, dtype=np.int32)
    fn = _lib.oracle_topk_qsort if use_qsort else _lib.oracle_topk
    rc = fn(_p(v), _p(i), _p(score), score.shape[-1], k)
    if rc:
        raise ValueError("oracle_topk rc=%d" % rc)
    return v, i


def swiglu(mlp1_out, limit=7.0):
    mlp1_out = _f32(mlp1_out)
    I = mlp1_out.shape[-1] // 2
    out = np.empty(I, dtype=np.float32)
    _lib.oracle_swiglu(_p(out), _p(mlp1_out), I, limit)
    return out


def moe_block(t, w_router, b_router, w_mlp1, b_mlp1, w_mlp2, b_mlp2, K, swiglu_limit=7.0, want_scores=False):
    """All weights fp32 (how the reference CPU path holds them).  Returns e_agg, topk_i, topk_v[, scores]."""
    t = _f32(t)
    T, H = t.shape
    E = w_router.shape[0]
    I = w_mlp2.shape[-1]
    arrs = [_f32(a) for a in (w_router, b_router, w_mlp1, b_mlp1, w_mlp2, b_mlp2)]
    assert arrs[2].shape == (E, 2 * I, H) and arrs[4].shape == (E, H, I)
    e_agg = np.empty((T, H), dtype=np.float32)
    topk_i = np.empty((T, K), dtype=np.int32)
    topk_v = np.empty((T, K), dtype=np.float32)
    scores = np.empty((T, E), dtype=np.float32) if want_scores else None
    rc = _lib.oracle_moe_block(T, H, I, E, K, swiglu_limit, _p(t), *[_p(a) for a in arrs], _p(e_agg), _p(topk_i),
                               _p(topk_v), _p(scores))
    if rc:
        raise ValueError("oracle_moe_block rc=%d" % rc)
    return (e_agg, topk_i, topk_v, scores) if want_scores else (e_agg, topk_i, topk_v)


def moe_layer(x, rms_w, w_router, b_router, w_mlp1, b_mlp1, w_mlp2, b_mlp2, K, swiglu_limit=7.0):
    """x <- x + moe_block(rmsnorm(x)) ; returns (x_out, topk_i, topk_v)."""
    x = _f32(x).copy()
    T, H = x.shape
    E = w_router.shape[0]
    I = w_mlp2.shape[-1]
    arrs = [_f32(a) for a in (rms_w, w_router, b_router, w_mlp1, b_mlp1, w_mlp2, b_mlp2)]
    t_s = np.empty((T, H), dtype=np.float32)
    a_s = np.empty((T, H), dtype=np.float32)
    topk_i = np.empty((T, K), dtype=np.int32)
    topk_v = np.empty((T, K), dtype=np.float32)
    rc = _lib.oracle_moe_layer(T, H, I, E, K, swiglu_limit, _p(x), *[_p(a) for a in arrs], _p(t_s), _p(a_s),
                               _p(topk_i), _p(topk_v))
    if rc:
        raise ValueError("oracle_moe_layer rc=%d" % rc)
    return x, topk_i, topk_v


def mxfp4_to_bf16_bits(code, scale):
    return int(_lib.oracle_mxfp4_to_bf16_bits(code, scale))


def dequant_mxfp4(blocks, scales):
    """blocks [...,G,16] u8, scales [...,G] u8 -> bf16 bit patterns (uint16) [..., G*32]."""
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    scales = np.ascontiguousarray(scales, dtype=np.uint8)
    assert blocks.shape[:-1] == scales.shape and blocks.shape[-1] == 16
    out = np.empty(scales.shape[:-1] + (scales.shape[-1] * 32,), dtype=np.uint16)
    _lib.oracle_dequant_mxfp4(_p(blocks), _p(scales), scales.size, _p(out))
    return out


def dequant_mxfp4_f32(blocks, scales, out=None):
    """dequant_mxfp4 widened to fp32 in the same pass; `out` (C-contiguous fp32 of the result's size) is filled in
    place when given."""
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    scales = np.ascontiguousarray(scales, dtype=np.uint8)
    assert blocks.shape[:-1] == scales.shape and blocks.shape[-1] == 16
    if out is None:
        out = np.empty(scales.shape[:-1] + (scales.shape[-1] * 32,), dtype=np.float32)
    assert out.dtype == np.float32 and out.flags.c_contiguous and out.size == scales.size * 32
    _lib.oracle_dequant_mxfp4_f32(_p(blocks), _p(scales), scales.size, _p(out))
    return out


def bf16_to_f32(bits, out=None):
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    if out is None:
        out = np.empty(bits.shape, dtype=np.float32)
    assert out.dtype == np.float32 and out.flags.c_contiguous and out.size == bits.size
    _lib.oracle_bf16_to_f32(_p(bits), bits.size, _p(out))
    return out


def f32_to_bf16(x):
    x = _f32(x)
    out = np.empty(x.shape, dtype=np.uint16)
    _lib.oracle_f32_to_bf16(_p(x), x.size, _p(out))
    return out


def bucket(topk_i, topk_v, E):
    topk_i = np.ascontiguousarray(topk_i, dtype=np.int32)
    topk_v = _f32(topk_v)
    T, K = topk_i.shape
    offsets = np.empty(E + 1, dtype=np.int32)
    tokens_flat = np.empty(T * K, dtype=np.int32)
    weights_flat = np.empty(T * K, dtype=np.float32)
    slot_of = np.empty(T * K, dtype=np.int32)
    rc = _lib.oracle_bucket(_p(topk_i), _p(topk_v), T, K, E, _p(offsets), _p(tokens_flat), _p(weights_flat),
                            _p(slot_of))
    if rc:
        raise ValueError("oracle_bucket rc=%d" % rc)
    return offsets, tokens_flat, weights_flat, slot_of.reshape(T, K)


def classify_queues(expert_offsets, very_sparse_cutoff, heavy_factor_sparse, heavy_factor_default):
    """(wq_heavy [n_heavy, 3], wq_light [n_light, 3], stats) with stats = (heavy_count, light_count,
    heavy_maxNe, active_experts, sumNe)."""
    off = np.ascontiguousarray(expert_offsets, dtype=np.int32)
    E = len(off) - 1
    wq_h = np.full(3 * E, -1, dtype=np.int32)
    wq_l = np.full(3 * E, -1, dtype=np.int32)
    stats = np.zeros(5, dtype=np.int64)
    _lib.oracle_classify_queues(_p(off), E, very_sparse_cutoff, heavy_factor_sparse, heavy_factor_default, _p(wq_h),
                                _p(wq_l), _p(stats))
    return wq_h[: 3 * stats[0]].reshape(-1, 3), wq_l[: 3 * stats[1]].reshape(-1, 3), tuple(int(v) for v in stats)


# ---- synthetic inputs (include/moe_synth.h), host side ------------------------------------------
_TABLE = None


def normal_table():
    global _TABLE
    if _TABLE is None:
        t = np.empty(1 << 16, dtype=np.float32)
        _lib.oracle_synth_normal_table(_p(t))
        _TABLE = t
    return _TABLE


def synth_normal_f32(shape, scale, seed, tensor_id, start=0):
    """Elements start .. start+prod(shape)-1 of the stream (seed, tensor_id)."""
    out = np.empty(shape, dtype=np.float32)
    _lib.oracle_synth_normal_f32(_p(out), out.size, _p(normal_table()), scale, seed, tensor_id, start)
    return out


def synth_normal_bf16(shape, scale, seed, tensor_id, start=0):
    out = np.empty(shape, dtype=np.uint16)
    _lib.oracle_synth_normal_bf16(_p(out), out.size, _p(normal_table()), scale, seed, tensor_id, start)
    return out


def synth_bytes(shape, seed, tensor_id, start=0):
    out = np.empty(shape, dtype=np.uint8)
    _lib.oracle_synth_bytes(_p(out), out.size, seed, tensor_id, start)
    return out


def synth_range_bytes(shape, seed, tensor_id, lo, span, start=0):
    out = np.empty(shape, dtype=np.uint8)
    _lib.oracle_synth_range_bytes(_p(out), out.size, seed, tensor_id, lo, span, start)
    return out
