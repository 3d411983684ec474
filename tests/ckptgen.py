"""Writers of tiny synthetic checkpoints in the two on-disk formats the reader takes.

They are the test-side statement of the formats, written from the reference's exporter
(tools/model_export/gpt-oss-20b/export_model_bin.py): the .bin is the fifteen config fields in
KEYS order (:33-49, :232-241) followed by every tensor, grouped by the CATEGORIES suffix list in
its order and by layer index inside a group (:51-71, :203-227), as fp32 or raw bf16 (:244-268);
the safetensors file is that exporter's input, experts as `.blocks`/`.scales` (:150-196).
"""
import json
import re
import struct

import numpy as np

CONFIG_KEYS = ["vocab_size", "hidden_size", "num_experts", "experts_per_token", "intermediate_size",
               "num_hidden_layers", "head_dim", "num_attention_heads", "num_key_value_heads", "max_seq_len",
               "initial_context_length", "rope_theta", "rope_scaling_factor", "sliding_window", "swiglu_limit"]

SUFFIX_ORDER = ["embedding.weight", "unembedding.weight", "attn.norm.scale", "mlp.norm.scale", "norm.scale",
                "attn.qkv.weight", "attn.qkv.bias", "attn.out.weight", "attn.out.bias", "attn.sinks",
                "mlp.gate.weight", "mlp.gate.bias", "mlp.mlp1_weight", "mlp.mlp1_bias", "mlp.mlp2_weight",
                "mlp.mlp2_bias"]

TINY = dict(vocab_size=11, hidden_size=64, num_experts=4, experts_per_token=2, intermediate_size=32,
            num_hidden_layers=3, head_dim=8, num_attention_heads=4, num_key_value_heads=2, max_seq_len=16,
            initial_context_length=32, rope_theta=150000.0, rope_scaling_factor=32.0, sliding_window=8,
            swiglu_limit=7.0)


def f32_to_bf16_bits(a):
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def bf16_bits_to_f32(b):
    return (b.astype(np.uint32) << 16).view(np.float32)


def mxfp4_dequant(blocks, scales):
    """fp32 values (all bf16-representable here) of blocks [..., G, 16] / scales [..., G]."""
    lut = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0., -.5, -1, -1.5, -2, -3, -4, -6], dtype=np.float32)
    out = np.empty(blocks.shape[:-1] + (32,), dtype=np.float32)
    out[..., 0::2] = lut[blocks & 0xF]
    out[..., 1::2] = lut[blocks >> 4]
    out *= np.exp2(scales.astype(np.float32) - 127)[..., None]
    return out.reshape(blocks.shape[:-2] + (blocks.shape[-2] * 32,))


def make_tensors(cfg, seed, mxfp4):
    """name -> array for a whole tiny model.  Dense values are bf16-representable fp32; with
    `mxfp4` the expert weights are `.blocks`/`.scales` u8 pairs instead."""
    rng = np.random.default_rng(seed)
    V, H, E, I, L = (cfg[k] for k in ("vocab_size", "hidden_size", "num_experts", "intermediate_size",
                                      "num_hidden_layers"))
    hd, nq, nkv = cfg["head_dim"], cfg["num_attention_heads"], cfg["num_key_value_heads"]
    qkv = hd * nq + 2 * hd * nkv

    def dense(*shape, scale=1.0):
        return bf16_bits_to_f32(f32_to_bf16_bits(rng.standard_normal(shape) * scale))

    t = {"embedding.weight": dense(V, H), "unembedding.weight": dense(V, H), "norm.scale": dense(H)}
    for l in range(L):
        p = "block.%d." % l
        t[p + "attn.norm.scale"] = dense(H)
        t[p + "mlp.norm.scale"] = dense(H)
        t[p + "attn.qkv.weight"] = dense(qkv, H)
        t[p + "attn.qkv.bias"] = dense(qkv)
        t[p + "attn.out.weight"] = dense(H, hd * nq)
        t[p + "attn.out.bias"] = dense(H)
        t[p + "attn.sinks"] = dense(nq)
        t[p + "mlp.gate.weight"] = dense(E, H, scale=0.3)
        t[p + "mlp.gate.bias"] = dense(E, scale=0.1)
        t[p + "mlp.mlp1_bias"] = dense(E, 2 * I, scale=0.1)
        t[p + "mlp.mlp2_bias"] = dense(E, H, scale=0.1)
        if mxfp4:
            t[p + "mlp.mlp1_weight.blocks"] = rng.integers(0, 256, (E, 2 * I, H // 32, 16), dtype=np.uint8)
            t[p + "mlp.mlp1_weight.scales"] = rng.integers(120, 127, (E, 2 * I, H // 32), dtype=np.uint8)
            t[p + "mlp.mlp2_weight.blocks"] = rng.integers(0, 256, (E, H, I // 32, 16), dtype=np.uint8)
            t[p + "mlp.mlp2_weight.scales"] = rng.integers(120, 127, (E, H, I // 32), dtype=np.uint8)
        else:
            t[p + "mlp.mlp1_weight"] = dense(E, 2 * I, H, scale=0.1)
            t[p + "mlp.mlp2_weight"] = dense(E, H, I, scale=0.1)
    return t


def bin_order(names):
    groups = {s: [] for s in SUFFIX_ORDER}
    rest = []
    for n in names:
        for s in SUFFIX_ORDER:
            if n.endswith(s):
                m = re.search(r"block\.(\d+)\.", n)
                groups[s].append((int(m.group(1)) if m else -1, n))
                break
        else:
            rest.append(n)
    return [n for s in SUFFIX_ORDER for _, n in sorted(groups[s])] + sorted(rest)


def write_bin(path, cfg, tensors, bf16=False):
    """`tensors` must be dense (name -> fp32 array)."""
    with open(path, "wb") as f:
        for k in CONFIG_KEYS:
            f.write(struct.pack("<i" if isinstance(cfg[k], int) else "<f", cfg[k]))
        for n in bin_order(list(tensors)):
            a = np.ascontiguousarray(tensors[n], dtype=np.float32)
            f.write((f32_to_bf16_bits(a) if bf16 else a).tobytes())


def write_safetensors(path, tensors, bf16_names=(), metadata=None, pad_header=0, extra_keys=False):
    """Hand-rolled writer (u64 header length, JSON header, data), so that the tests control the
    header text: key order, whitespace, `__metadata__`, unknown per-tensor keys.  fp32 arrays whose
    name is in `bf16_names` are stored as BF16."""
    header, blobs, at = {}, [], 0
    if metadata is not None:
        header["__metadata__"] = metadata
    for n, a in tensors.items():
        if a.dtype == np.uint8:
            dt, raw = "U8", np.ascontiguousarray(a).tobytes()
        elif n in bf16_names:
            dt, raw = "BF16", f32_to_bf16_bits(a).tobytes()
        else:
            dt, raw = "F32", np.ascontiguousarray(a, dtype=np.float32).tobytes()
        entry = {"dtype": dt, "shape": list(a.shape), "data_offsets": [at, at + len(raw)]}
        if extra_keys:
            entry = {"note": {"nested": [1, 2.5e3, True, None, "x\\\"y"]}, **entry}
        header[n] = entry
        blobs.append(raw)
        at += len(raw)
    text = json.dumps(header, indent=1 if extra_keys else None).encode() + b" " * pad_header
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text)))
        f.write(text)
        for b in blobs:
            f.write(b)
