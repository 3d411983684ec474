"""ctypes binding of the checkpoint reader declared in include/moe_checkpoint.h: the reference's
packed .bin (src/run.cpp:196-283) and safetensors files with MXFP4 experts
(tools/model_export/gpt-oss-20b/export_model_bin.py:150-196), uploaded one layer at a time into
the device layouts of moe_block_forward.  File parsing and the upload run in the C++ library;
torch only provides the device buffers.
"""
import ctypes

import numpy as np
import torch

from . import (MOE_WEIGHTS_BF16, MOE_WEIGHTS_MXFP4_TILED, MoeBlock, MoeError, _check, _ptr, _stream, lib,
               mxfp4_tiled_bytes)

_c = ctypes
_vp, _i, _sz = _c.c_void_p, _c.c_int, _c.c_size_t

DTYPE_F32, DTYPE_BF16, DTYPE_U8, DTYPE_OTHER = 0, 1, 2, 3
(T_RMS_FFN, T_W_ROUTER, T_B_ROUTER, T_W_MLP1, T_B_MLP1, T_W_MLP2, T_B_MLP2, T_W_MLP1_SCALES,
 T_W_MLP2_SCALES) = range(9)
_NP = {DTYPE_F32: np.float32, DTYPE_BF16: np.uint16, DTYPE_U8: np.uint8, DTYPE_OTHER: np.uint8}


class CkptConfig(_c.Structure):
    """moe_ckpt_config: the reference's Config (src/run.cpp:26-46), field for field."""
    _fields_ = [(n, _c.c_int32) for n in (
        "vocab_size", "hidden_dim", "n_experts", "experts_per_token", "intermediate_dim", "n_layers", "head_dim",
        "n_attn_heads", "n_kv_heads", "seq_len", "initial_context_length")] + [
        ("rope_theta", _c.c_float), ("rope_scaling_factor", _c.c_float), ("sliding_window", _c.c_int32),
        ("swiglu_limit", _c.c_float)]


class LayerDevice(_c.Structure):
    """moe_layer_device of include/moe_checkpoint.h."""
    _fields_ = [("struct_bytes", _c.c_uint32), ("weight_format", _c.c_int32), ("rms_ffn_w", _vp), ("w_router", _vp),
                ("b_router", _vp), ("w_mlp1", _vp), ("w_mlp1_scales", _vp), ("b_mlp1", _vp), ("w_mlp2", _vp),
                ("w_mlp2_scales", _vp), ("b_mlp2", _vp)]


# name -> (restype, argtypes); every symbol include/moe_checkpoint.h declares
SIGNATURES = {
    "moe_ckpt_open_bin": (_i, [_c.c_char_p, _i, _c.POINTER(_vp)]),
    "moe_ckpt_open_safetensors": (_i, [_c.c_char_p, _c.POINTER(CkptConfig), _c.POINTER(_vp)]),
    "moe_ckpt_close": (None, [_vp]),
    "moe_ckpt_get_config": (_i, [_vp, _c.POINTER(CkptConfig)]),
    "moe_ckpt_is_mxfp4": (_i, [_vp]),
    "moe_ckpt_layer_tensor": (_i, [_vp, _i, _i, _c.POINTER(_vp), _c.POINTER(_sz), _c.POINTER(_i)]),
    "moe_ckpt_n_tensors": (_i, [_vp]),
    "moe_ckpt_tensor_info": (_i, [_vp, _i, _c.POINTER(_c.c_char_p), _c.POINTER(_i), _c.POINTER(_i),
                                  _c.POINTER(_c.c_longlong), _c.POINTER(_vp), _c.POINTER(_sz)]),
    "moe_ckpt_staging_bytes": (_sz, [_vp]),
    "moe_ckpt_upload_layer": (_i, [_vp, _i, _c.POINTER(LayerDevice), _vp, _sz, _vp]),
}
for _name, (_res, _args) in SIGNATURES.items():
    _fn = getattr(lib, _name)
    _fn.restype, _fn.argtypes = _res, _args


class Checkpoint:
    """An open checkpoint file (read-only memory map owned by the library)."""

    def __init__(self, handle):
        self._h = handle
        cfg = CkptConfig()
        _check("moe_ckpt_get_config", lib.moe_ckpt_get_config(self._h, ctypes.byref(cfg)))
        self.config = cfg
        self.is_mxfp4 = bool(lib.moe_ckpt_is_mxfp4(self._h))

    @classmethod
    def open_bin(cls, path, payload_dtype=DTYPE_F32):
        h = _vp()
        _check("moe_ckpt_open_bin", lib.moe_ckpt_open_bin(str(path).encode(), payload_dtype, ctypes.byref(h)))
        return cls(h)

    @classmethod
    def open_safetensors(cls, path, config=None):
        h = _vp()
        cfg = ctypes.byref(config) if config is not None else None
        _check("moe_ckpt_open_safetensors", lib.moe_ckpt_open_safetensors(str(path).encode(), cfg, ctypes.byref(h)))
        return cls(h)

    def close(self):
        if self._h:
            lib.moe_ckpt_close(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        self.close()

    def _view(self, ptr, nbytes, dtype):
        buf = (ctypes.c_uint8 * nbytes).from_address(ptr.value)
        return np.frombuffer(buf, dtype=_NP[dtype]).copy()

    def layer_tensor(self, layer, which):
        """(flat numpy copy, dtype code) of one MoE tensor; bf16 comes back as its uint16 bit patterns."""
        p, n, d = _vp(), _sz(), _i()
        _check("moe_ckpt_layer_tensor",
               lib.moe_ckpt_layer_tensor(self._h, layer, which, ctypes.byref(p), ctypes.byref(n), ctypes.byref(d)))
        return self._view(p, n.value, d.value), d.value

    def tensors(self):
        """[(name, dtype code, shape, nbytes)] of every tensor the reader indexed."""
        out = []
        for i in range(lib.moe_ckpt_n_tensors(self._h)):
            name, d, r, n = _c.c_char_p(), _i(), _i(), _sz()
            shape = (_c.c_longlong * 8)()
            _check("moe_ckpt_tensor_info", lib.moe_ckpt_tensor_info(
                self._h, i, ctypes.byref(name), ctypes.byref(d), ctypes.byref(r), shape, None, ctypes.byref(n)))
            out.append((name.value.decode(), d.value, tuple(shape[:r.value]), n.value))
        return out

    def staging_bytes(self):
        return lib.moe_ckpt_staging_bytes(self._h)

    def upload_layer(self, layer, device="cuda", tiled=None, staging=None, stream=None, with_norm=True):
        """Allocates the device tensors of one layer and fills them from the file.  Returns a dict
        with the MoeBlock constructor's weight arguments plus `rms_ffn_w`.  `tiled` defaults to
        True for MXFP4 files (weights stay 4-bit in HBM)."""
        c = self.config
        H, I, E = c.hidden_dim, c.intermediate_dim, c.n_experts
        tiled = self.is_mxfp4 if tiled is None else tiled
        u16 = dict(dtype=torch.uint16, device=device)
        t = dict(w_router=torch.empty((E, H), **u16), b_router=torch.empty((E,), **u16),
                 b_mlp1=torch.empty((E, 2 * I), **u16), b_mlp2=torch.empty((E, H), **u16),
                 rms_ffn_w=torch.empty((H,), **u16) if with_norm else None)
        if tiled:
            u8 = dict(dtype=torch.uint8, device=device)
            b1, s1 = mxfp4_tiled_bytes(2 * I, H)
            b2, s2 = mxfp4_tiled_bytes(H, I)
            if b1 == 0 or b2 == 0:
                raise MoeError("moe_mxfp4_tiled_bytes", -2)
            t.update(w_mlp1=torch.empty(E * b1, **u8), w_mlp1_scales=torch.empty(E * s1, **u8),
                     w_mlp2=torch.empty(E * b2, **u8), w_mlp2_scales=torch.empty(E * s2, **u8))
        else:
            t.update(w_mlp1=torch.empty((E, 2 * I, H), **u16), w_mlp2=torch.empty((E, H, I), **u16),
                     w_mlp1_scales=None, w_mlp2_scales=None)
        if staging is None:
            staging = torch.empty(max(self.staging_bytes(), 64 << 20), dtype=torch.uint8, device=device)
        d = LayerDevice()
        d.struct_bytes = ctypes.sizeof(LayerDevice)
        d.weight_format = MOE_WEIGHTS_MXFP4_TILED if tiled else MOE_WEIGHTS_BF16
        for k, v in t.items():
            setattr(d, k, _ptr(v))
        _check("moe_ckpt_upload_layer", lib.moe_ckpt_upload_layer(
            self._h, layer, ctypes.byref(d), _ptr(staging), staging.numel(), _stream(stream)))
        torch.cuda.synchronize()  # the staging buffer and the file map are free to go after this
        return t

    def moe_block(self, layer, max_tokens, device="cuda", tiled=None):
        """MoeBlock over layer `layer`'s weights, with K and the SwiGLU limit from the file's config."""
        t = self.upload_layer(layer, device=device, tiled=tiled, with_norm=False)
        t.pop("rms_ffn_w")
        c = self.config
        return MoeBlock(c.hidden_dim, c.intermediate_dim, c.n_experts, c.experts_per_token, max_tokens=max_tokens,
                        swiglu_limit=c.swiglu_limit, **t)
