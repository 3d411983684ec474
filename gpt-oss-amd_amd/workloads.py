"""Synthetic MoE workloads: shapes, tensor streams and device-side generation.

Every tensor is a pure function of (seed, tensor_id, index) (include/moe_synth.h), so the same
description drives the device generator here and a host generator elsewhere and both produce the
same bits.  Shapes follow the reference's checkpoints
(tools/model_export/gpt-oss-20b/config.json, tools/model_export/gpt-oss-120b/config.json).
"""
import dataclasses
import math

import numpy as np
import torch

import importlib

_pkg = importlib.import_module(__package__)

# tensor stream ids (include/moe_synth.h)
TID_X, TID_W_ROUTER, TID_B_ROUTER, TID_W_MLP1, TID_B_MLP1, TID_W_MLP2, TID_B_MLP2 = 1, 2, 3, 4, 5, 6, 7
TID_W_MLP1_SCALES, TID_W_MLP2_SCALES, TID_RANK_PERM = 8, 9, 10
LAYER_STRIDE = 16

ZIPF_BETA = 0.515  # bias = beta * (-s * ln rank): realised top-1 histogram has log-log slope ~ -s


@dataclasses.dataclass(frozen=True)
class MoeShape:
    name: str
    T: int                 # tokens
    H: int = 2880          # hidden
    I: int = 2880          # expert intermediate
    E: int = 32            # experts
    K: int = 4             # experts per token
    fmt: str = "bf16"      # "bf16" | "mxfp4"
    zipf_s: float = 0.0    # > 0: router bias gives Zipf(s)-skewed expert load
    layers: int = 1
    seed: int = 0
    swiglu_limit: float = 7.0
    alpha: float = 1.702


WORKLOADS = {
    "cpu64_bf16": MoeShape("cpu64_bf16", T=64),
    "decode256_bf16": MoeShape("decode256_bf16", T=256),
    "decode256_mxfp4": MoeShape("decode256_mxfp4", T=256, fmt="mxfp4"),
    "prefill4096_mxfp4_zipf": MoeShape("prefill4096_mxfp4_zipf", T=4096, fmt="mxfp4", zipf_s=1.2),
    "prefill4096_bf16": MoeShape("prefill4096_bf16", T=4096),
    "layer120b_mxfp4": MoeShape("layer120b_mxfp4", T=1024, E=128, fmt="mxfp4"),
    "stack120b_mxfp4": MoeShape("stack120b_mxfp4", T=1024, E=128, fmt="mxfp4", layers=36),
}


def synth_hash(seed, tensor_id, idx):
    """moe_synth_hash of include/moe_synth.h in Python integers."""
    m = (1 << 64) - 1
    z = (idx + 0x9E3779B97F4A7C15 * (((seed << 20) + tensor_id + 1) & m)) & m
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & m
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & m
    z = z ^ (z >> 31)
    return z >> 32


def f32_to_bf16_bits(x):
    """Round-to-nearest-even fp32 -> bf16 bit patterns (numpy, finite inputs)."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF).astype(np.uint16)


def zipf_router_bias_bits(shape, layer=0):
    """bf16 bits of b[e] = beta * (-s * ln rank(e)), rank = permutation seeded per layer."""
    keys = [synth_hash(shape.seed, TID_RANK_PERM + LAYER_STRIDE * layer, e) for e in range(shape.E)]
    order = sorted(range(shape.E), key=lambda e: (keys[e], e))
    rank = np.empty(shape.E, dtype=np.int64)
    for r, e in enumerate(order):
        rank[e] = r + 1
    b = (ZIPF_BETA * (-shape.zipf_s * np.log(rank.astype(np.float64)))).astype(np.float32)
    return f32_to_bf16_bits(b)


def tensor_specs(shape, layer=0):
    """name -> (dims, kind, args).  kinds: normal_f32(scale), normal_bf16(scale), bytes,
    range_bytes(lo, span), host_bf16(bits array)."""
    o = LAYER_STRIDE * layer
    H, I, E = shape.H, shape.I, shape.E
    s = {
        "w_router": ((E, H), "normal_bf16", (0.02, TID_W_ROUTER + o)),
        "b_mlp1": ((E, 2 * I), "normal_bf16", (0.02, TID_B_MLP1 + o)),
        "b_mlp2": ((E, H), "normal_bf16", (0.02, TID_B_MLP2 + o)),
    }
    if shape.zipf_s > 0:
        s["b_router"] = ((E,), "host_bf16", (zipf_router_bias_bits(shape, layer),))
    else:
        s["b_router"] = ((E,), "normal_bf16", (0.02, TID_B_ROUTER + o))
    if shape.fmt == "bf16":
        s["w_mlp1"] = ((E, 2 * I, H), "normal_bf16", (0.02, TID_W_MLP1 + o))
        s["w_mlp2"] = ((E, H, I), "normal_bf16", (0.02, TID_W_MLP2 + o))
    else:
        s["w_mlp1_blocks"] = ((E, 2 * I, H // 32, 16), "bytes", (TID_W_MLP1 + o,))
        s["w_mlp1_scales"] = ((E, 2 * I, H // 32), "range_bytes", (TID_W_MLP1_SCALES + o, 119, 9))
        s["w_mlp2_blocks"] = ((E, H, I // 32, 16), "bytes", (TID_W_MLP2 + o,))
        s["w_mlp2_scales"] = ((E, H, I // 32), "range_bytes", (TID_W_MLP2_SCALES + o, 119, 9))
    return s


def input_spec(shape):
    return ((shape.T, shape.H), "normal_f32", (1.0, TID_X))


_TABLE_CACHE = {}


def normal_table_device(table_host, device):
    key = (str(device), table_host.ctypes.data)
    if key not in _TABLE_CACHE:
        _TABLE_CACHE[key] = torch.from_numpy(table_host).to(device)
    return _TABLE_CACHE[key]


def fill_device(dims, kind, args, seed, table_d, device):
    """Generate one tensor in device memory."""
    if kind == "normal_f32":
        t = torch.empty(dims, dtype=torch.float32, device=device)
        _pkg.synth_normal_f32(t, table_d, args[0], seed, args[1])
    elif kind == "normal_bf16":
        t = torch.empty(dims, dtype=torch.bfloat16, device=device)
        _pkg.synth_normal_bf16(t, table_d, args[0], seed, args[1])
    elif kind == "bytes":
        t = torch.empty(dims, dtype=torch.uint8, device=device)
        _pkg.synth_bytes(t, seed, args[0])
    elif kind == "range_bytes":
        t = torch.empty(dims, dtype=torch.uint8, device=device)
        _pkg.synth_range_bytes(t, seed, args[0], args[1], args[2])
    elif kind == "host_bf16":
        t = torch.from_numpy(args[0].view(np.int16).copy()).view(torch.bfloat16).to(device)
    else:
        raise ValueError(kind)
    return t


def make_device_layer(shape, table_host, device, layer=0, keep_canonical=False, workspace=None):
    """Weights of one layer in device memory, MXFP4 tensors repacked to the tiled layout.
    Returns (MoeBlock, dict of raw tensors)."""
    table_d = normal_table_device(table_host, device)
    raw = {n: fill_device(d, k, a, shape.seed, table_d, device) for n, (d, k, a) in tensor_specs(shape, layer).items()}
    if shape.fmt == "bf16":
        blk = _pkg.MoeBlock(shape.H, shape.I, shape.E, shape.K, raw["w_router"], raw["b_router"], raw["w_mlp1"],
                            raw["b_mlp1"], raw["w_mlp2"], raw["b_mlp2"], max_tokens=shape.T,
                            swiglu_limit=shape.swiglu_limit, alpha=shape.alpha, workspace=workspace)
    else:
        t1b, t1s = _pkg.mxfp4_repack(raw["w_mlp1_blocks"], raw["w_mlp1_scales"])
        t2b, t2s = _pkg.mxfp4_repack(raw["w_mlp2_blocks"], raw["w_mlp2_scales"])
        blk = _pkg.MoeBlock(shape.H, shape.I, shape.E, shape.K, raw["w_router"], raw["b_router"], t1b, raw["b_mlp1"],
                            t2b, raw["b_mlp2"], max_tokens=shape.T, w_mlp1_scales=t1s, w_mlp2_scales=t2s,
                            swiglu_limit=shape.swiglu_limit, alpha=shape.alpha, workspace=workspace)
        if not keep_canonical:
            torch.cuda.synchronize(device)
            for n in ("w_mlp1_blocks", "w_mlp1_scales", "w_mlp2_blocks", "w_mlp2_scales"):
                del raw[n]
    return blk, raw


def make_device_input(shape, table_host, device):
    d, k, a = input_spec(shape)
    return fill_device(d, k, a, shape.seed, normal_table_device(table_host, device), device)


class DeviceStack:
    """shape.layers MoE layers resident in device memory with the reference's layer glue around each
    block: t = rmsnorm(x) with unit weight (src/forward.cpp:315), x += moe(t) (src/forward.cpp:514)."""

    def __init__(self, shape, table_host, device):
        self.shape = shape
        nbytes = _pkg.block_workspace_bytes(shape.T, shape.H, shape.I, shape.E, shape.K)
        self.workspace = torch.empty(nbytes, dtype=torch.uint8, device=device)
        self.blocks = []
        for layer in range(shape.layers):
            blk, raw = make_device_layer(shape, table_host, device, layer=layer, workspace=self.workspace)
            del raw
            self.blocks.append(blk)
        self.rms_w = torch.ones(shape.H, dtype=torch.bfloat16, device=device)
        T = shape.T
        self.t = torch.empty((T, shape.H), dtype=torch.float32, device=device)
        self.e_agg = torch.empty((T, shape.H), dtype=torch.float32, device=device)
        self.topk_i = torch.empty((shape.layers, T, shape.K), dtype=torch.int32, device=device)
        self.topk_v = torch.empty((shape.layers, T, shape.K), dtype=torch.float32, device=device)

    def prepare(self, x):
        """Parameter blocks for forward(x): built once so the timed loop does no Python tensor work."""
        # every block but the last also produces the next layer's normalised input (fused into its combine)
        last = len(self.blocks) - 1
        self.params = [blk.params(self.t, self.e_agg, self.topk_i[l], self.topk_v[l], residual_x=x,
                                  next_norm_weight=None if l == last else self.rms_w,
                                  next_norm_out=None if l == last else self.t)
                       for l, blk in enumerate(self.blocks)]
        self.packed = _pkg.pack_layer_params(self.params)
        self.x = x

    def forward(self, stream=None, start=0, stop=None):
        """x <- x + moe_l(rmsnorm(x)) for l = start .. stop-1 (all layers by default), in place on self.x."""
        s = torch.cuda.current_stream().cuda_stream if stream is None else stream
        T, H = self.shape.T, self.shape.H
        stop = len(self.blocks) if stop is None else stop
        _pkg.rmsnorm(self.t, self.x, self.rms_w, T, H, stream=s)  # later layers get theirs from the block before
        # one call issues all the layers: nothing of the host language sits between two layers' launches
        if stop > start:
            _pkg.forward_layers(self.packed, s, start, stop - start)


# ---- algorithmic work per block (what roofline fractions are computed from) ----------------------
def weight_bytes_per_expert(shape):
    H, I = shape.H, shape.I
    if shape.fmt == "bf16":
        return (2 * I * H + H * I) * 2
    return (2 * I * H + H * I) // 2 + (2 * I * H + H * I) // 32


def algorithmic_bytes(shape, active_experts=None):
    """Each active expert's weights and biases once, router weights once, block input and output
    once; intermediates are implementation traffic and are not counted."""
    E_act = shape.E if active_experts is None else active_experts
    H, I, E, T = shape.H, shape.I, shape.E, shape.T
    bias_bytes = (2 * I + H) * 2
    return E_act * (weight_bytes_per_expert(shape) + bias_bytes) + E * H * 2 + E * 2 + 2 * T * H * 4


def algorithmic_flops(shape):
    H, I, E, T, K = shape.H, shape.I, shape.E, shape.T, shape.K
    return K * T * 2 * (2 * I * H + H * I) + 2 * T * H * E
