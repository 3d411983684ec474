"""ctypes binding of libmoe_gfx950.so — the gpt-oss MoE expert block for one MI355X (gfx950).

The functions here carry the names and argument order of the reference's host-callable kernels
(src/hip/gemms/gemm_router.hip:184, src/hip/topk.hip:59, src/hip/softmax.hip:46,
src/hip/moe.hip:237 and :514, src/hip/vecadd.hip:32) and pass torch device tensors straight
through to the C ABI declared in include/moe_abi.h.  torch is used for device memory and streams
only; all arithmetic runs in the HIP library.  There is no CPU fallback: if the library has not
been built, importing this package raises.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# MOE_GFX950_LIB selects another build of the same library (A/B timing of two builds in one session)
LIB_PATH = os.environ.get("MOE_GFX950_LIB") or os.path.join(_HERE, "libmoe_gfx950.so")

MOE_WEIGHTS_BF16 = 0
MOE_WEIGHTS_MXFP4_TILED = 1
MOE_FLAG_ROUTER_STRICT_ORDER = 1
MOE_FLAG_FORCE_STREAM = 2
MOE_FLAG_FORCE_TILED = 4
MOE_FLAG_FORCE_DIRECT = 8
MOE_FLAG_FORCE_BUCKET_LAUNCH = 16
MOE_FLAG_FUSED_GEMM_LAUNCH = 32

_c = ctypes
_vp, _i, _ll, _f, _u, _sz = _c.c_void_p, _c.c_int, _c.c_longlong, _c.c_float, _c.c_uint, _c.c_size_t


class MoeError(RuntimeError):
    def __init__(self, fn, code):
        msg = _lib.moe_error_string(code).decode()
        super().__init__("%s failed: %s (code %d)" % (fn, msg, code))
        self.code = code


class BlockParams(_c.Structure):
    """moe_block_params of include/moe_abi.h."""
    _fields_ = [
        ("struct_bytes", _c.c_uint32),
        ("n_tokens", _c.c_int32),
        ("hidden_dim", _c.c_int32),
        ("intermediate_dim", _c.c_int32),
        ("n_experts", _c.c_int32),
        ("experts_per_token", _c.c_int32),
        ("weight_format", _c.c_int32),
        ("swiglu_limit", _f),
        ("alpha", _f),
        ("t", _vp),
        ("w_router", _vp),
        ("b_router", _vp),
        ("w_mlp1", _vp),
        ("w_mlp1_scales", _vp),
        ("b_mlp1", _vp),
        ("w_mlp2", _vp),
        ("w_mlp2_scales", _vp),
        ("b_mlp2", _vp),
        ("e_agg", _vp),
        ("topk_i", _vp),
        ("topk_v", _vp),
        ("router_score", _vp),
        ("residual_x", _vp),
        ("workspace", _vp),
        ("workspace_bytes", _sz),
        ("flags", _c.c_uint32),
        ("next_norm_weight", _vp),
        ("next_norm_out", _vp),
    ]


# name -> (restype, argtypes); every symbol include/moe_abi.h declares
SIGNATURES = {
    "moe_abi_version": (_i, []),
    "moe_error_string": (_c.c_char_p, [_i]),
    "moe_router_scratch_bytes": (_sz, [_i, _i]),
    "moe_gemm_router": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp, _sz, _vp]),
    "moe_gemm_router_static_max_bytes": (_sz, []),
    "moe_gemm_router_static": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "moe_router_two_pass_scratch_bytes": (_sz, [_i, _i, _i]),
    "moe_router_two_pass_report": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _vp, _sz, _vp, _vp, _vp, _vp, _vp, _vp]),
    "moe_topk": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "moe_softmax": (_i, [_vp, _i, _i, _vp]),
    "moe_bucket_by_expert": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp, _vp, _vp, _vp]),
    "moe_gather_rows": (_i, [_vp, _vp, _vp, _i, _i, _vp]),
    "moe_scatter_rows": (_i, [_vp, _vp, _vp, _i, _i, _vp]),
    "moe_build_work_queue": (_i, [_vp, _i, _vp, _vp, _vp]),
    "moe_count_tokens_per_expert": (_i, [_vp, _vp, _i, _i, _vp, _vp, _vp, _vp, _i, _vp]),
    "moe_exclusive_scan_expert_offsets": (_i, [_vp, _vp, _i, _vp]),
    "moe_compact_by_expert": (_i, [_vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _i, _vp]),
    "moe_classify_and_build_queues": (_i, [_vp, _i, _i, _f, _f, _vp, _vp, _vp, _vp]),
    "moe_mlp1_swiglu": (_i, [_vp, _i, _i, _vp, _vp, _vp, _vp, _i, _i, _ll, _ll, _f, _f, _i, _i, _vp]),
    "moe_mlp2_scatter": (_i, [_vp, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _ll, _ll, _i, _i, _vp]),
    "moe_mlp1_swiglu_mxfp4": (_i, [_vp, _i, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _ll, _f, _f, _i, _i, _vp]),
    "moe_mlp2_scatter_mxfp4": (_i, [_vp, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _ll, _i, _i, _vp]),
    "moe_vecadd_and_zero": (_i, [_vp, _vp, _f, _i, _i, _vp]),
    "moe_rmsnorm": (_i, [_vp, _vp, _vp, _i, _i, _vp]),
    "moe_dequant_mxfp4": (_i, [_vp, _vp, _ll, _vp, _vp]),
    "moe_mxfp4_tiled_bytes": (None, [_i, _i, _c.POINTER(_sz), _c.POINTER(_sz)]),
    "moe_mxfp4_repack": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp, _vp]),
    "moe_mxfp4_unpack": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp, _vp]),
    "moe_mxfp4_tiled_to_bf16": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp]),
    "moe_block_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "moe_block_forward": (_i, [_c.POINTER(BlockParams), _vp]),
    "moe_block_forward_layers": (_i, [_vp, _i, _vp]),
    "moe_block_describe": (_i, [_c.POINTER(BlockParams), _c.c_char_p, _sz]),
    "moe_synth_normal_table": (None, [_vp]),
    "moe_block_down_gemm": (_i, [_c.POINTER(BlockParams), _vp, _vp, _vp]),
    "moe_stage_timer_create": (_i, [_c.POINTER(_vp)]),
    "moe_stage_timer_destroy": (None, [_vp]),
    "moe_block_forward_timed": (_i, [_c.POINTER(BlockParams), _vp, _vp]),
    "moe_stage_timer_read": (_i, [_vp, _c.POINTER(_f)]),
    "moe_synth_normal_f32": (_i, [_vp, _ll, _vp, _f, _u, _u, _vp]),
    "moe_synth_normal_bf16": (_i, [_vp, _ll, _vp, _f, _u, _u, _vp]),
    "moe_synth_bytes": (_i, [_vp, _ll, _u, _u, _vp]),
    "moe_synth_range_bytes": (_i, [_vp, _ll, _u, _u, _u, _u, _vp]),
    "moe_synth_checksum": (_i, [_vp, _ll, _vp, _vp]),
    "moe_device_attributes": (_i, [_vp, _vp, _vp, _vp, _vp]),
}


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "%s is missing: build it with `python gpt-oss-amd_amd/build.py` (hipcc, gfx950). "
            "There is no CPU fallback for the MoE kernels." % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here = a declared symbol is not exported
        fn.restype = res
        fn.argtypes = args
    return lib


_lib = _load()
lib = _lib


def _ptr(t):
    if t is None:
        return None
    if isinstance(t, int):
        return t
    if not t.is_cuda:
        raise ValueError("expected a device tensor")
    if not t.is_contiguous():
        raise ValueError("expected a contiguous tensor")
    return t.data_ptr()


def _stream(stream):
    if stream is None:
        return torch.cuda.current_stream().cuda_stream
    return stream.cuda_stream if hasattr(stream, "cuda_stream") else stream


def _check(fn, rc):
    if rc != 0:
        raise MoeError(fn, rc)


# ---- reference-named entry points --------------------------------------------------------------
def gemm_router(xout, x_batch, w, bias, N, K, M, stream=None, scratch=None):
    """src/hip/gemms/gemm_router.hip:184 — xout[N,M] = x_batch[N,K] @ w[M,K]^T + bias[M]."""
    if scratch is None:
        scratch = torch.empty(_lib.moe_router_scratch_bytes(N, M), dtype=torch.uint8, device=xout.device)
    _check("moe_gemm_router", _lib.moe_gemm_router(_ptr(xout), _ptr(x_batch), _ptr(w), _ptr(bias), N, K, M,
                                                   _ptr(scratch), scratch.numel(), _stream(stream)))


def gemm_router_static(xout, x_batch, w, bias, N, K, M, stream=None):
    """gemm_router with the reference's exact argument list; scratch is a fixed array inside the library,
    nothing is allocated (N * M limited: moe_gemm_router_static in include/moe_abi.h)."""
    _check("moe_gemm_router_static", _lib.moe_gemm_router_static(_ptr(xout), _ptr(x_batch), _ptr(w), _ptr(bias), N, K,
                                                                 M, _stream(stream)))


def router_two_pass_report(x, w, bias, K, stream=None):
    """The two-pass router with its intermediate results: (topk_v, topk_i, approx_scores, bound, n_candidates)."""
    T, H = x.shape
    E = w.shape[0]
    dev = x.device
    scratch = torch.empty(_lib.moe_router_two_pass_scratch_bytes(T, H, E), dtype=torch.uint8, device=dev)
    tv = torch.empty((T, K), dtype=torch.float32, device=dev)
    ti = torch.empty((T, K), dtype=torch.int32, device=dev)
    approx = torch.empty((T, E), dtype=torch.float32, device=dev)
    bound = torch.empty((T,), dtype=torch.float32, device=dev)
    n_cand = torch.empty((T,), dtype=torch.int32, device=dev)
    _check("moe_router_two_pass_report",
           _lib.moe_router_two_pass_report(_ptr(x), _ptr(w), _ptr(bias), T, H, E, K, _ptr(scratch), scratch.numel(),
                                           _ptr(tv), _ptr(ti), _ptr(approx), _ptr(bound), _ptr(n_cand), _stream(stream)))
    return tv, ti, approx, bound, n_cand


def topk(topk_values, topk_indices, router_scores, batch_size, num_experts, experts_per_token, stream=None):
    """src/hip/topk.hip:59."""
    _check("moe_topk", _lib.moe_topk(_ptr(topk_values), _ptr(topk_indices), _ptr(router_scores), batch_size,
                                     num_experts, experts_per_token, _stream(stream)))


def softmax(x, batch_size, size, stream=None):
    """src/hip/softmax.hip:46 — in place."""
    _check("moe_softmax", _lib.moe_softmax(_ptr(x), batch_size, size, _stream(stream)))


def bucket_by_expert(topk_i, topk_v, B, K, E, expert_offsets, tokens_flat, weights_flat, slot_of=None, stream=None):
    """src/hip/scheduler.hip:11-61 in one launch (count, scan, compaction)."""
    _check("moe_bucket_by_expert",
           _lib.moe_bucket_by_expert(_ptr(topk_i), _ptr(topk_v), B, K, E, _ptr(expert_offsets), _ptr(tokens_flat),
                                     _ptr(weights_flat), _ptr(slot_of), _stream(stream)))


def count_tokens_per_expert(topk_i, topk_v, B, K, out_expert, out_token, out_w, counts, E, stream=None):
    """count_tokens_per_expert of src/hip/scheduler.hip:11-31 (counts must be zero on entry)."""
    _check("moe_count_tokens_per_expert",
           _lib.moe_count_tokens_per_expert(_ptr(topk_i), _ptr(topk_v), B, K, _ptr(out_expert), _ptr(out_token),
                                            _ptr(out_w), _ptr(counts), E, _stream(stream)))


def exclusive_scan_expert_offsets(counts, offsets, E, stream=None):
    """exclusive_scan_expert_offsets of src/hip/scheduler.hip:33-46 (zeroes counts)."""
    _check("moe_exclusive_scan_expert_offsets",
           _lib.moe_exclusive_scan_expert_offsets(_ptr(counts), _ptr(offsets), E, _stream(stream)))


def compact_by_expert(expert_ids, tokens, weights, BK, offsets, write_counters, tokens_flat, weights_flat, E,
                      stream=None):
    """compact_by_expert_kernel of src/hip/scheduler.hip:48-61, buckets in ascending assignment index."""
    _check("moe_compact_by_expert",
           _lib.moe_compact_by_expert(_ptr(expert_ids), _ptr(tokens), _ptr(weights), BK, _ptr(offsets),
                                      _ptr(write_counters), _ptr(tokens_flat), _ptr(weights_flat), E, _stream(stream)))


def classify_and_build_queues(expert_offsets, E, very_sparse_cutoff, heavy_factor_sparse, heavy_factor_default,
                              wq_heavy, wq_light, stats, stream=None):
    """classify_and_build_queues of src/hip/scheduler.hip:112-184; `stats` is a device buffer of 24 bytes
    (four int32 and one int64: heavy_count, light_count, heavy_maxNe, active_experts, sumNe)."""
    _check("moe_classify_and_build_queues",
           _lib.moe_classify_and_build_queues(_ptr(expert_offsets), E, very_sparse_cutoff, heavy_factor_sparse,
                                              heavy_factor_default, _ptr(wq_heavy), _ptr(wq_light), _ptr(stats),
                                              _stream(stream)))


def gather_rows(X, idx, Y, rows, H, stream=None):
    """src/hip/scheduler.hip:63-85."""
    _check("moe_gather_rows", _lib.moe_gather_rows(_ptr(X), _ptr(idx), _ptr(Y), rows, H, _stream(stream)))


def scatter_rows(Y, idx, X, rows, H, stream=None):
    """X[idx[row], :] = Y[row, :] (inverse of gather_rows)."""
    _check("moe_scatter_rows", _lib.moe_scatter_rows(_ptr(Y), _ptr(idx), _ptr(X), rows, H, _stream(stream)))


def build_work_queue(expert_offsets, E, work_queue, work_count, stream=None):
    """src/hip/scheduler.hip:112-184 (single queue)."""
    _check("moe_build_work_queue",
           _lib.moe_build_work_queue(_ptr(expert_offsets), E, _ptr(work_queue), _ptr(work_count), _stream(stream)))


def moe_mlp1_swiglu(work_queue, work_start, work_count, x_by_expert, gate_by_expert, weights_base, bias_base, H, I,
                    expert_weight_stride, expert_bias_stride, alpha, swiglu_limit, maxNe, grid_cap, stream=None):
    """src/hip/moe.hip:237."""
    _check("moe_mlp1_swiglu",
           _lib.moe_mlp1_swiglu(_ptr(work_queue), work_start, work_count, _ptr(x_by_expert), _ptr(gate_by_expert),
                                _ptr(weights_base), _ptr(bias_base), H, I, expert_weight_stride, expert_bias_stride,
                                alpha, swiglu_limit, maxNe, grid_cap, _stream(stream)))


def moe_mlp2_scatter(work_queue, work_start, work_count, gate_by_expert, tokens_flat, weights_flat, e_agg,
                     weights_base, bias_base, I, H, expert_weight_stride, expert_bias_stride, maxNe, grid_cap,
                     stream=None):
    """src/hip/moe.hip:514."""
    _check("moe_mlp2_scatter",
           _lib.moe_mlp2_scatter(_ptr(work_queue), work_start, work_count, _ptr(gate_by_expert), _ptr(tokens_flat),
                                 _ptr(weights_flat), _ptr(e_agg), _ptr(weights_base), _ptr(bias_base), I, H,
                                 expert_weight_stride, expert_bias_stride, maxNe, grid_cap, _stream(stream)))


def moe_mlp1_swiglu_mxfp4(work_queue, work_start, work_count, x_by_expert, gate_by_expert, tiled_blocks,
                          tiled_scales, bias_base, H, I, expert_bias_stride, alpha, swiglu_limit, maxNe, grid_cap,
                          stream=None):
    _check("moe_mlp1_swiglu_mxfp4",
           _lib.moe_mlp1_swiglu_mxfp4(_ptr(work_queue), work_start, work_count, _ptr(x_by_expert),
                                      _ptr(gate_by_expert), _ptr(tiled_blocks), _ptr(tiled_scales), _ptr(bias_base),
                                      H, I, expert_bias_stride, alpha, swiglu_limit, maxNe, grid_cap,
                                      _stream(stream)))


def moe_mlp2_scatter_mxfp4(work_queue, work_start, work_count, gate_by_expert, tokens_flat, weights_flat, e_agg,
                           tiled_blocks, tiled_scales, bias_base, I, H, expert_bias_stride, maxNe, grid_cap,
                           stream=None):
    _check("moe_mlp2_scatter_mxfp4",
           _lib.moe_mlp2_scatter_mxfp4(_ptr(work_queue), work_start, work_count, _ptr(gate_by_expert),
                                       _ptr(tokens_flat), _ptr(weights_flat), _ptr(e_agg), _ptr(tiled_blocks),
                                       _ptr(tiled_scales), _ptr(bias_base), I, H, expert_bias_stride, maxNe,
                                       grid_cap, _stream(stream)))


def vecadd_and_zero(a, b, weight, batch, size, stream=None):
    """src/hip/vecadd.hip:32."""
    _check("moe_vecadd_and_zero", _lib.moe_vecadd_and_zero(_ptr(a), _ptr(b), weight, batch, size, _stream(stream)))


def rmsnorm(o, x, weight, batch, size, stream=None):
    """src/hip/rmsnorm.hip:39 (batched)."""
    _check("moe_rmsnorm", _lib.moe_rmsnorm(_ptr(o), _ptr(x), _ptr(weight), batch, size, _stream(stream)))


# ---- MXFP4 -------------------------------------------------------------------------------------
def dequant_mxfp4(blocks, scales, out=None, stream=None):
    """blocks [..., G, 16] u8, scales [..., G] u8 -> bf16 [..., G*32]
    (tools/model_export/gpt-oss-20b/export_model_bin.py:95-133)."""
    n_blocks = scales.numel()
    if out is None:
        out = torch.empty(tuple(scales.shape[:-1]) + (scales.shape[-1] * 32,), dtype=torch.bfloat16,
                          device=blocks.device)
    _check("moe_dequant_mxfp4", _lib.moe_dequant_mxfp4(_ptr(blocks), _ptr(scales), n_blocks, _ptr(out),
                                                       _stream(stream)))
    return out


def mxfp4_tiled_bytes(rows, K):
    bb, sb = _sz(0), _sz(0)
    _lib.moe_mxfp4_tiled_bytes(rows, K, ctypes.byref(bb), ctypes.byref(sb))
    return bb.value, sb.value


def mxfp4_repack(blocks, scales, stream=None, out=None):
    """blocks [E, rows, G, 16], scales [E, rows, G] -> (tiled_blocks, tiled_scales) u8 tensors (`out`: a pair of
    u8 tensors of E * moe_mxfp4_tiled_bytes to fill instead of new ones)."""
    E, rows, G = scales.shape
    bb, sb = mxfp4_tiled_bytes(rows, G * 32)
    if bb == 0:
        raise MoeError("moe_mxfp4_tiled_bytes", -2)
    if out is not None:
        tb, ts = out
        assert tb.numel() == E * bb and ts.numel() == E * sb and tb.dtype == ts.dtype == torch.uint8
    else:
        tb = torch.empty(E * bb, dtype=torch.uint8, device=blocks.device)
        ts = torch.empty(E * sb, dtype=torch.uint8, device=blocks.device)
    _check("moe_mxfp4_repack", _lib.moe_mxfp4_repack(_ptr(blocks), _ptr(scales), E, rows, G * 32, _ptr(tb), _ptr(ts),
                                                     _stream(stream)))
    return tb, ts


def mxfp4_unpack(tiled_blocks, tiled_scales, E, rows, K, stream=None):
    G = K // 32
    blocks = torch.empty((E, rows, G, 16), dtype=torch.uint8, device=tiled_blocks.device)
    scales = torch.empty((E, rows, G), dtype=torch.uint8, device=tiled_blocks.device)
    _check("moe_mxfp4_unpack", _lib.moe_mxfp4_unpack(_ptr(tiled_blocks), _ptr(tiled_scales), E, rows, K, _ptr(blocks),
                                                     _ptr(scales), _stream(stream)))
    return blocks, scales


def mxfp4_tiled_to_bf16(tiled_blocks, tiled_scales, E, rows, K, stream=None):
    out = torch.empty((E, rows, K), dtype=torch.bfloat16, device=tiled_blocks.device)
    _check("moe_mxfp4_tiled_to_bf16", _lib.moe_mxfp4_tiled_to_bf16(_ptr(tiled_blocks), _ptr(tiled_scales), E, rows, K,
                                                                   _ptr(out), _stream(stream)))
    return out


# ---- whole block -------------------------------------------------------------------------------
def block_workspace_bytes(T, H, I, E, K):
    return _lib.moe_block_workspace_bytes(T, H, I, E, K)


class MoeBlock:
    """One layer's MoE weights plus a workspace sized for up to `max_tokens`; `forward` runs
    router -> top-k -> softmax -> bucketing -> experts -> combine (src/forward.cpp:317-514)."""

    def __init__(self, H, I, E, K, w_router, b_router, w_mlp1, b_mlp1, w_mlp2, b_mlp2, max_tokens,
                 w_mlp1_scales=None, w_mlp2_scales=None, swiglu_limit=7.0, alpha=1.702, workspace=None):
        self.H, self.I, self.E, self.K = H, I, E, K
        self.fmt = MOE_WEIGHTS_BF16 if w_mlp1_scales is None else MOE_WEIGHTS_MXFP4_TILED
        self.tensors = dict(w_router=w_router, b_router=b_router, w_mlp1=w_mlp1, b_mlp1=b_mlp1, w_mlp2=w_mlp2,
                            b_mlp2=b_mlp2, w_mlp1_scales=w_mlp1_scales, w_mlp2_scales=w_mlp2_scales)
        self.swiglu_limit, self.alpha = swiglu_limit, alpha
        self.max_tokens = max_tokens
        nbytes = block_workspace_bytes(max_tokens, H, I, E, K)
        if nbytes == 0:
            raise MoeError("moe_block_workspace_bytes", -2)
        if workspace is None:
            workspace = torch.empty(nbytes, dtype=torch.uint8, device=w_router.device)
        elif workspace.numel() < nbytes:
            raise MoeError("moe_block_workspace_bytes", -4)
        self.workspace = workspace  # layers run one after another on a stream may share it

    def params(self, t, e_agg, topk_i, topk_v, router_score=None, residual_x=None, flags=0, next_norm_weight=None,
               next_norm_out=None):
        T = t.shape[0] if t is not None else topk_i.shape[0]
        p = BlockParams()
        p.struct_bytes = ctypes.sizeof(BlockParams)
        p.n_tokens, p.hidden_dim, p.intermediate_dim = T, self.H, self.I
        p.n_experts, p.experts_per_token, p.weight_format = self.E, self.K, self.fmt
        p.swiglu_limit, p.alpha = self.swiglu_limit, self.alpha
        p.t = _ptr(t)
        for k, v in self.tensors.items():
            setattr(p, k, _ptr(v))
        p.e_agg, p.topk_i, p.topk_v = _ptr(e_agg), _ptr(topk_i), _ptr(topk_v)
        p.router_score, p.residual_x = _ptr(router_score), _ptr(residual_x)
        p.workspace, p.workspace_bytes = _ptr(self.workspace), self.workspace.numel()
        p.flags = flags
        p.next_norm_weight, p.next_norm_out = _ptr(next_norm_weight), _ptr(next_norm_out)
        return p

    def forward(self, t, e_agg=None, topk_i=None, topk_v=None, router_score=None, residual_x=None, flags=0,
                stream=None, next_norm_weight=None, next_norm_out=None):
        T = t.shape[0]
        dev = t.device
        if e_agg is None:
            e_agg = torch.empty((T, self.H), dtype=torch.float32, device=dev)
        if topk_i is None:
            topk_i = torch.empty((T, self.K), dtype=torch.int32, device=dev)
        if topk_v is None:
            topk_v = torch.empty((T, self.K), dtype=torch.float32, device=dev)
        p = self.params(t, e_agg, topk_i, topk_v, router_score, residual_x, flags, next_norm_weight, next_norm_out)
        _check("moe_block_forward", _lib.moe_block_forward(ctypes.byref(p), _stream(stream)))
        return e_agg, topk_i, topk_v

    def down_gemm(self, topk_i, h_by_assignment, flags=0, stream=None):
        """The block's down-projection GEMM alone: bf16 rows [T*K, I] by assignment -> fp32 rows [T*K, H]."""
        T = topk_i.shape[0]
        y = torch.empty((T * self.K, self.H), dtype=torch.float32, device=topk_i.device)
        tv = torch.ones((T, self.K), dtype=torch.float32, device=topk_i.device)
        p = self.params(None, None, topk_i, tv, flags=flags)
        p.n_tokens = T
        _check("moe_block_down_gemm", _lib.moe_block_down_gemm(ctypes.byref(p), _ptr(h_by_assignment), _ptr(y),
                                                               _stream(stream)))
        return y

    def describe(self, p):
        """Which kernels moe_block_forward launches for parameter block p: dict of the 'key=value' parts."""
        buf = ctypes.create_string_buffer(1024)
        _check("moe_block_describe", _lib.moe_block_describe(ctypes.byref(p), buf, len(buf)))
        return dict(part.split("=", 1) for part in buf.value.decode().split("; "))

    def launch(self, p, stream):
        """Re-issue a prepared parameter block (benchmark loop: no Python-side tensor work)."""
        rc = _lib.moe_block_forward(ctypes.byref(p), stream)
        if rc:
            raise MoeError("moe_block_forward", rc)


def pack_layer_params(params):
    """A ctypes array holding copies of the parameter blocks of consecutive layers, for forward_layers()."""
    arr = (BlockParams * len(params))()
    for i, p in enumerate(params):
        ctypes.memmove(ctypes.byref(arr, i * ctypes.sizeof(BlockParams)), ctypes.byref(p), ctypes.sizeof(BlockParams))
    return arr


def forward_layers(packed, stream, start=0, count=None):
    """moe_block_forward_layers: layers start .. start+count-1 of a pack_layer_params() array in one call."""
    n = len(packed) - start if count is None else count
    _check("moe_block_forward_layers",
           _lib.moe_block_forward_layers(ctypes.byref(packed, start * ctypes.sizeof(BlockParams)), n, stream))


STAGES = ("router_partial", "router_finalize", "bucket", "mlp1_swiglu", "mlp2", "combine")


class StageTimer:
    """HIP-event timer for the six stages of moe_block_forward (moe_stage_timer of the C ABI)."""

    def __init__(self):
        self._h = _vp()
        _check("moe_stage_timer_create", _lib.moe_stage_timer_create(ctypes.byref(self._h)))

    def launch(self, p, stream):
        _check("moe_block_forward_timed", _lib.moe_block_forward_timed(ctypes.byref(p), stream, self._h))

    def read(self):
        out = (_f * len(STAGES))()
        _check("moe_stage_timer_read", _lib.moe_stage_timer_read(self._h, out))
        return list(out)

    def close(self):
        if self._h:
            _lib.moe_stage_timer_destroy(self._h)
            self._h = _vp()

    def __del__(self):
        self.close()


# ---- synthetic workloads (include/moe_synth.h) --------------------------------------------------
def normal_table():
    """The generator's table of N(0,1) quantiles (numpy float32 [65536]), built by the library."""
    import numpy as np
    table = np.empty(1 << 16, dtype=np.float32)
    _lib.moe_synth_normal_table(table.ctypes.data)
    return table



def synth_normal_f32(dst, table_d, scale, seed, tensor_id, stream=None):
    _check("moe_synth_normal_f32", _lib.moe_synth_normal_f32(_ptr(dst), dst.numel(), _ptr(table_d), scale, seed,
                                                             tensor_id, _stream(stream)))


def synth_normal_bf16(dst, table_d, scale, seed, tensor_id, stream=None):
    _check("moe_synth_normal_bf16", _lib.moe_synth_normal_bf16(_ptr(dst), dst.numel(), _ptr(table_d), scale, seed,
                                                               tensor_id, _stream(stream)))


def synth_bytes(dst, seed, tensor_id, stream=None):
    _check("moe_synth_bytes", _lib.moe_synth_bytes(_ptr(dst), dst.numel(), seed, tensor_id, _stream(stream)))


def device_attributes():
    """dict of what the current device reports: compute_units, clock_khz, memory_clock_khz, memory_bus_bits, l2_bytes."""
    vals = [_c.c_int(0) for _ in range(5)]
    _check("moe_device_attributes", _lib.moe_device_attributes(*[ctypes.byref(v) for v in vals]))
    return dict(zip(("compute_units", "clock_khz", "memory_clock_khz", "memory_bus_bits", "l2_bytes"), [v.value for v in vals]))


SYNTH_CHECKSUM_WORDS = 2049


def synth_checksum(src, out=None, stream=None):
    """Launches the checksum of `src` (any dtype, byte size a multiple of 16); returns the int64 device tensor whose
    element 0 is the sum of the buffer's 32-bit words modulo 2^64 once the stream has run."""
    import torch
    if out is None:
        out = torch.empty(SYNTH_CHECKSUM_WORDS, dtype=torch.int64, device=src.device)
    _check("moe_synth_checksum", _lib.moe_synth_checksum(_ptr(src), src.numel() * src.element_size(), _ptr(out),
                                                         _stream(stream)))
    return out


def synth_range_bytes(dst, seed, tensor_id, lo, span, stream=None):
    _check("moe_synth_range_bytes", _lib.moe_synth_range_bytes(_ptr(dst), dst.numel(), seed, tensor_id, lo, span,
                                                               _stream(stream)))
