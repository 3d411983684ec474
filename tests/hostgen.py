"""Host-side generation of the synthetic workloads (same streams as the device generator of
gpt_oss_amd_amd.workloads) and conversion to what the CPU oracle consumes (fp32 weights)."""
import numpy as np


def host_tensor(oracle, dims, kind, args, seed, start=0):
    if kind == "normal_f32":
        return oracle.synth_normal_f32(dims, args[0], seed, args[1], start)
    if kind == "normal_bf16":
        return oracle.synth_normal_bf16(dims, args[0], seed, args[1], start)  # uint16 bit patterns
    if kind == "bytes":
        return oracle.synth_bytes(dims, seed, args[0], start)
    if kind == "range_bytes":
        return oracle.synth_range_bytes(dims, seed, args[0], args[1], args[2], start)
    if kind == "host_bf16":
        assert start == 0
        return args[0].copy()
    raise ValueError(kind)


def host_layer(oracle, wl, shape, layer=0, experts=None):
    """fp32 weights of one layer as the reference CPU path holds them.  `experts` restricts the
    (large) expert tensors to a subset: the arrays keep their full [E, ...] shape, but only the
    listed experts are generated (the rest stays untouched zero pages)."""
    specs = wl.tensor_specs(shape, layer)
    out = {}
    for name in ("w_router", "b_router", "b_mlp1", "b_mlp2"):
        d, k, a = specs[name]
        out[name] = oracle.bf16_to_f32(host_tensor(oracle, d, k, a, shape.seed))
    todo = range(shape.E) if experts is None else sorted(set(int(e) for e in experts))
    for name in ("w_mlp1", "w_mlp2"):
        if shape.fmt == "bf16":
            d, k, a = specs[name]
            per = int(np.prod(d[1:]))
            full = np.zeros(d, dtype=np.float32)
            for e in todo:
                oracle.bf16_to_f32(host_tensor(oracle, d[1:], k, a, shape.seed, start=e * per), out=full[e])
        else:
            db, kb, ab = specs[name + "_blocks"]
            ds, ks, as_ = specs[name + "_scales"]
            per_b, per_s = int(np.prod(db[1:])), int(np.prod(ds[1:]))
            full = np.zeros((db[0], db[1], db[2] * 32), dtype=np.float32)
            keep = experts is None
            if keep:
                out[name + "_blocks"] = np.empty(db, dtype=np.uint8)
                out[name + "_scales"] = np.empty(ds, dtype=np.uint8)
            for e in todo:
                blocks = host_tensor(oracle, db[1:], kb, ab, shape.seed, start=e * per_b)
                scales = host_tensor(oracle, ds[1:], ks, as_, shape.seed, start=e * per_s)
                oracle.dequant_mxfp4_f32(blocks, scales, out=full[e])
                if keep:
                    out[name + "_blocks"][e], out[name + "_scales"][e] = blocks, scales
        out[name] = full
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


def rms_err(y, ref):
    """||y - ref||_2 / ||ref||_2 : the RMS-relative error reported beside the tolerance metric."""
    d = y.astype(np.float64) - ref.astype(np.float64)
    return float(np.sqrt((d * d).sum() / (ref.astype(np.float64) ** 2).sum()))
