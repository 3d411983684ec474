"""Host-side generation of the synthetic workloads (same streams as the device generator of
gpt_oss_amd_amd.workloads) and conversion to what the CPU oracle consumes (fp32 weights)."""
import numpy as np


def host_tensor(oracle, dims, kind, args, seed):
    if kind == "normal_f32":
        return oracle.synth_normal_f32(dims, args[0], seed, args[1])
    if kind == "normal_bf16":
        return oracle.synth_normal_bf16(dims, args[0], seed, args[1])  # uint16 bit patterns
    if kind == "bytes":
        return oracle.synth_bytes(dims, seed, args[0])
    if kind == "range_bytes":
        return oracle.synth_range_bytes(dims, seed, args[0], args[1], args[2])
    if kind == "host_bf16":
        return args[0].copy()
    raise ValueError(kind)


def host_layer(oracle, wl, shape, layer=0, experts=None):
    """fp32 weights of one layer as the reference CPU path holds them.  `experts` restricts the
    (large) expert tensors to a subset: entries of other experts are left zero."""
    specs = wl.tensor_specs(shape, layer)
    out = {}
    for name in ("w_router", "b_router", "b_mlp1", "b_mlp2"):
        d, k, a = specs[name]
        out[name] = oracle.bf16_to_f32(host_tensor(oracle, d, k, a, shape.seed))
    if shape.fmt == "bf16":
        for name in ("w_mlp1", "w_mlp2"):
            d, k, a = specs[name]
            out[name] = oracle.bf16_to_f32(host_tensor(oracle, d, k, a, shape.seed))
    else:
        for name in ("w_mlp1", "w_mlp2"):
            d, k, a = specs[name + "_blocks"]
            blocks = host_tensor(oracle, d, k, a, shape.seed)
            d, k, a = specs[name + "_scales"]
            scales = host_tensor(oracle, d, k, a, shape.seed)
            out[name + "_blocks"], out[name + "_scales"] = blocks, scales
            out[name] = oracle.bf16_to_f32(oracle.dequant_mxfp4(blocks, scales))
    return out


def host_input(oracle, wl, shape):
    d, k, a = wl.input_spec(shape)
    return host_tensor(oracle, d, k, a, shape.seed)


def oracle_block(oracle, shape, hw, t):
    return oracle.moe_block(t, hw["w_router"], hw["b_router"], hw["w_mlp1"], hw["b_mlp1"], hw["w_mlp2"],
                            hw["b_mlp2"], shape.K, shape.swiglu_limit, want_scores=True)


def rel_err(y, ref):
    """max|y - ref| / max|ref| : the output tolerance metric (outputs cross zero, so an element-wise
    relative error has no meaning)."""
    return float(np.abs(y.astype(np.float64) - ref.astype(np.float64)).max() / np.abs(ref).max())
