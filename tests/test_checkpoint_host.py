"""Checkpoint reader (include/moe_checkpoint.h), host side: no GPU needed.  Tiny files in both
on-disk formats are written by tests/ckptgen.py and read back through the C ABI."""
import ctypes
import os
import re
import struct

import numpy as np
import pytest

import ckptgen
from conftest import ROOT


@pytest.fixture(scope="module")
def ck(pkg):
    import importlib
    return importlib.import_module("gpt_oss_amd_amd.checkpoint")


MOE_NAMES = ["mlp.norm.scale", "mlp.gate.weight", "mlp.gate.bias", "mlp.mlp1_weight", "mlp.mlp1_bias",
             "mlp.mlp2_weight", "mlp.mlp2_bias"]


def test_header_symbols_exported(pkg, ck):
    text = open(os.path.join(ROOT, "include", "moe_checkpoint.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(moe_ckpt_[a-z0-9_]+)\s*\(", text)))
    assert len(names) == 10
    raw = ctypes.CDLL(pkg.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), n
    assert sorted(ck.SIGNATURES) == names
    for code in (-7, -8, -9):
        assert len(pkg.lib.moe_error_string(code)) > 10
    assert ctypes.sizeof(ck.CkptConfig) == 60


@pytest.mark.parametrize("bf16", [False, True])
def test_bin_layout(ck, tmp_path, bf16):
    cfg = ckptgen.TINY
    tensors = ckptgen.make_tensors(cfg, seed=3, mxfp4=False)
    path = tmp_path / "model.bin"
    ckptgen.write_bin(path, cfg, tensors, bf16=bf16)
    with ck.Checkpoint.open_bin(path, ck.DTYPE_BF16 if bf16 else ck.DTYPE_F32) as c:
        got = c.config
        for key, field in zip(ckptgen.CONFIG_KEYS, [f[0] for f in ck.CkptConfig._fields_]):
            assert getattr(got, field) == cfg[key], key
        assert not c.is_mxfp4
        assert len(c.tensors()) == 7 * cfg["num_hidden_layers"]
        for l in range(cfg["num_hidden_layers"]):
            for which, name in enumerate(MOE_NAMES):
                want = tensors["block.%d.%s" % (l, name)].ravel()
                data, dtype = c.layer_tensor(l, which)
                if bf16:
                    assert dtype == ck.DTYPE_BF16 and np.array_equal(data, ckptgen.f32_to_bf16_bits(want))
                else:
                    assert dtype == ck.DTYPE_F32 and np.array_equal(data, want)
            with pytest.raises(Exception) as e:
                c.layer_tensor(l, ck.T_W_MLP1_SCALES)
            assert e.value.code == -9
        names = [t[0] for t in c.tensors()]
        assert names[0] == "block.0.mlp.norm.scale" and names[-1] == "block.2.mlp.mlp2_bias"
        shapes = {t[0]: t[2] for t in c.tensors()}
        assert shapes["block.1.mlp.mlp1_weight"] == (4, 64, 64) and shapes["block.1.mlp.mlp2_weight"] == (4, 64, 32)


def test_bin_rejects_wrong_files(ck, tmp_path):
    cfg = ckptgen.TINY
    tensors = ckptgen.make_tensors(cfg, seed=4, mxfp4=False)
    path = tmp_path / "model.bin"
    ckptgen.write_bin(path, cfg, tensors)
    raw = open(path, "rb").read()

    def code_of(data, dtype=ck.DTYPE_F32, name="bad.bin"):
        p = tmp_path / name
        open(p, "wb").write(data)
        with pytest.raises(Exception) as e:
            ck.Checkpoint.open_bin(p, dtype)
        return e.value.code

    assert code_of(raw[:-4]) == -2               # one float short
    assert code_of(raw + b"\0\0\0\0") == -2      # one float long
    assert code_of(raw, ck.DTYPE_BF16) == -2     # wrong payload width
    assert code_of(raw[:40]) == -8               # header cut short
    assert code_of(struct.pack("<i", -5) + raw[4:]) == -8   # nonsense config
    assert code_of(raw, dtype=7) == -5
    # every field inside its own limit, but the tensor sizes multiply out past 63 bits: a parse error,
    # not an offset that wrapped around to something that happens to match the file size
    huge = dict(cfg, vocab_size=1 << 24, hidden_size=1 << 20, num_experts=4096, experts_per_token=4,
                intermediate_size=1 << 20, num_hidden_layers=4096, head_dim=4096, num_attention_heads=4096,
                num_key_value_heads=4096)
    header = b"".join(struct.pack("<i" if isinstance(huge[k], int) else "<f", huge[k]) for k in ckptgen.CONFIG_KEYS)
    assert code_of(header + raw[len(header):]) == -8
    assert code_of(header) == -8
    with pytest.raises(Exception) as e:
        ck.Checkpoint.open_bin(tmp_path / "does_not_exist.bin")
    assert e.value.code == -7


@pytest.mark.parametrize("fancy", [False, True])
def test_safetensors_mxfp4(ck, tmp_path, fancy):
    cfg = ckptgen.TINY
    tensors = ckptgen.make_tensors(cfg, seed=5, mxfp4=True)
    bf16_names = {n for n in tensors if n.endswith("bias") or n.endswith("gate.weight")}
    path = tmp_path / "model.safetensors"
    ckptgen.write_safetensors(path, tensors, bf16_names, metadata={"format": "pt", "k": "v é"} if fancy else None,
                              pad_header=5 if fancy else 0, extra_keys=fancy)
    with ck.Checkpoint.open_safetensors(path) as c:
        assert c.is_mxfp4
        g = c.config
        assert (g.hidden_dim, g.intermediate_dim, g.n_experts, g.n_layers) == (64, 32, 4, 3)
        assert g.experts_per_token == 0  # not recorded in the file
        listed = {t[0]: t for t in c.tensors()}
        assert set(listed) == set(tensors)
        for n, a in tensors.items():
            assert listed[n][2] == a.shape
        for l in range(3):
            p = "block.%d.mlp." % l
            for which, name in ((ck.T_W_MLP1, "mlp1_weight.blocks"), (ck.T_W_MLP1_SCALES, "mlp1_weight.scales"),
                                (ck.T_W_MLP2, "mlp2_weight.blocks"), (ck.T_W_MLP2_SCALES, "mlp2_weight.scales")):
                data, dtype = c.layer_tensor(l, which)
                assert dtype == ck.DTYPE_U8 and np.array_equal(data, tensors[p + name].ravel())
            data, dtype = c.layer_tensor(l, ck.T_B_MLP1)
            assert dtype == ck.DTYPE_BF16 and np.array_equal(data, ckptgen.f32_to_bf16_bits(tensors[p + "mlp1_bias"]).ravel())
            data, dtype = c.layer_tensor(l, ck.T_RMS_FFN)
            assert dtype == ck.DTYPE_F32 and np.array_equal(data, tensors[p + "norm.scale"])
    # the same file read by the safetensors package, when it is importable: same names and bytes
    st = pytest.importorskip("safetensors")
    with st.safe_open(str(path), framework="np") as f:
        assert set(f.keys()) == set(tensors)
        assert np.array_equal(f.get_tensor("block.1.mlp.mlp2_weight.blocks"), tensors["block.1.mlp.mlp2_weight.blocks"])


GOLDEN = os.path.join(ROOT, "tests", "golden")
REF_CFG = dict(ckptgen.TINY, hidden_size=128, intermediate_size=64, num_experts=8, num_hidden_layers=2)


def ref_expected():
    """What tests/golden/make_ref_bin.py fed the reference's exporter: the same generator, config and seed."""
    tensors = ckptgen.make_tensors(REF_CFG, seed=11, mxfp4=True)
    dense = {}
    for n, a in tensors.items():
        if n.endswith(".scales"):
            continue
        if n.endswith(".blocks"):
            base = n[:-len(".blocks")]
            dense[base] = ckptgen.mxfp4_dequant(a, tensors[base + ".scales"])
        else:
            dense[n] = a
    return tensors, dense


@pytest.mark.parametrize("bf16", [False, True])
def test_reference_written_bin(ck, oracle, bf16):
    """tests/golden/ref_tiny_{f32,bf16}.bin were written by the reference's own export_model_bin.py (its
    dequantize_fp4, key order and header) from tests/golden/ref_tiny.safetensors.  The reader must find the
    reference's config in the header and every MoE tensor at the offset the exporter put it, and the expert values
    the exporter dequantised must be the ones the oracle's and the test generator's MXFP4 decoders give."""
    import json
    cfg = json.load(open(os.path.join(GOLDEN, "ref_tiny_config.json")))
    assert cfg == REF_CFG
    tensors, dense = ref_expected()
    path = os.path.join(GOLDEN, "ref_tiny_bf16.bin" if bf16 else "ref_tiny_f32.bin")
    raw = np.fromfile(path, dtype=np.uint8)
    width = 2 if bf16 else 4
    with ck.Checkpoint.open_bin(path, ck.DTYPE_BF16 if bf16 else ck.DTYPE_F32) as c:
        got = c.config
        for key, field in zip(ckptgen.CONFIG_KEYS, [f[0] for f in ck.CkptConfig._fields_]):
            assert getattr(got, field) == cfg[key], key
        assert not c.is_mxfp4 and len(c.tensors()) == 7 * 2
        # the exporter's order, restated: header, then tensors grouped by kind with the layers in order inside
        # each kind, so that the offsets of the MoE tensors depend on every tensor before them
        offset = 4 * len(ckptgen.CONFIG_KEYS)
        offsets = {}
        for n in ckptgen.bin_order(list(dense)):
            offsets[n] = offset
            offset += dense[n].size * width
        assert offset == raw.size
        for l in range(2):
            for which, name in enumerate(MOE_NAMES):
                full = "block.%d.%s" % (l, name)
                want = np.ascontiguousarray(dense[full], dtype=np.float32).ravel()
                data, dtype = c.layer_tensor(l, which)
                if bf16:
                    assert dtype == ck.DTYPE_BF16 and np.array_equal(data, ckptgen.f32_to_bf16_bits(want)), full
                else:
                    assert dtype == ck.DTYPE_F32 and np.array_equal(data.view(np.uint32), want.view(np.uint32)), full
                at = offsets[full]
                assert np.array_equal(raw[at:at + want.size * width], np.ascontiguousarray(data).view(np.uint8)), full
    # the oracle's decoder against the values the reference's dequantize_fp4 wrote (fp32 file: nothing rounded)
    f32 = np.fromfile(os.path.join(GOLDEN, "ref_tiny_f32.bin"), dtype=np.uint8)
    offset = 4 * len(ckptgen.CONFIG_KEYS)
    for n in ckptgen.bin_order(list(dense)):
        size = dense[n].size * 4
        if n.endswith("mlp1_weight") or n.endswith("mlp2_weight"):
            ref_vals = f32[offset:offset + size].view(np.float32)
            bits = oracle.dequant_mxfp4(tensors[n + ".blocks"], tensors[n + ".scales"])
            assert np.array_equal(ckptgen.f32_to_bf16_bits(ref_vals), bits.ravel()), n
            assert np.array_equal(ckptgen.bf16_bits_to_f32(bits.ravel()), ref_vals), n
        offset += size


def test_reference_read_safetensors(ck):
    """The safetensors file the reference's exporter read (tests/golden/ref_tiny.safetensors) through this reader:
    same expert blocks and scales, dense tensors as BF16."""
    tensors, _ = ref_expected()
    with ck.Checkpoint.open_safetensors(os.path.join(GOLDEN, "ref_tiny.safetensors")) as c:
        assert c.is_mxfp4
        g = c.config
        assert (g.hidden_dim, g.intermediate_dim, g.n_experts, g.n_layers) == (128, 64, 8, 2)
        for l in range(2):
            p = "block.%d.mlp." % l
            for which, name in ((ck.T_W_MLP1, "mlp1_weight.blocks"), (ck.T_W_MLP1_SCALES, "mlp1_weight.scales"),
                                (ck.T_W_MLP2, "mlp2_weight.blocks"), (ck.T_W_MLP2_SCALES, "mlp2_weight.scales")):
                data, dtype = c.layer_tensor(l, which)
                assert dtype == ck.DTYPE_U8 and np.array_equal(data, tensors[p + name].ravel())
            for which, name in ((ck.T_RMS_FFN, "norm.scale"), (ck.T_B_MLP1, "mlp1_bias"), (ck.T_B_MLP2, "mlp2_bias")):
                data, dtype = c.layer_tensor(l, which)
                assert dtype == ck.DTYPE_BF16 and np.array_equal(data, ckptgen.f32_to_bf16_bits(tensors[p + name]).ravel())


def test_safetensors_config_check_and_errors(ck, tmp_path):
    cfg = ckptgen.TINY
    tensors = ckptgen.make_tensors(cfg, seed=6, mxfp4=True)
    path = tmp_path / "m.safetensors"
    ckptgen.write_safetensors(path, tensors)
    want = ck.CkptConfig()
    want.experts_per_token, want.swiglu_limit, want.hidden_dim, want.n_layers = 2, 7.0, 64, 3
    with ck.Checkpoint.open_safetensors(path, want) as c:
        assert (c.config.experts_per_token, c.config.swiglu_limit, c.config.n_experts) == (2, 7.0, 4)
    want.hidden_dim = 128
    with pytest.raises(Exception) as e:
        ck.Checkpoint.open_safetensors(path, want)
    assert e.value.code == -2

    def code_of(tens=None, data=None):
        p = tmp_path / "bad.safetensors"
        if data is None:
            ckptgen.write_safetensors(p, tens)
        else:
            open(p, "wb").write(data)
        with pytest.raises(Exception) as e:
            ck.Checkpoint.open_safetensors(p)
        return e.value.code

    missing = {n: a for n, a in tensors.items() if n != "block.1.mlp.mlp2_weight.scales"}
    assert code_of(missing) == -9
    bad_shape = dict(tensors)
    bad_shape["block.2.mlp.mlp1_bias"] = np.zeros((4, 60), dtype=np.float32)
    assert code_of(bad_shape) == -2
    assert code_of({"embedding.weight": np.zeros((3, 4), dtype=np.float32)}) == -9  # no MoE layer at all
    raw = open(path, "rb").read()
    n = struct.unpack("<Q", raw[:8])[0]
    assert code_of(data=raw[:8 + n // 2]) == -8                       # header cut
    assert code_of(data=struct.pack("<Q", 1 << 40) + raw[8:]) == -8   # header length beyond the file
    assert code_of(data=raw[:-1]) == -8                                # last tensor runs past the end
    assert code_of(data=raw[:8] + raw[8:8 + n].replace(b'"U8"', b'"U9"', 1) + raw[8 + n:]) in (-2, -8)
    assert code_of(data=raw[:8] + b"[" + raw[9:]) == -8


def test_safetensors_dense(ck, tmp_path):
    cfg = ckptgen.TINY
    tensors = ckptgen.make_tensors(cfg, seed=7, mxfp4=False)
    path = tmp_path / "dense.safetensors"
    ckptgen.write_safetensors(path, tensors, bf16_names=set(tensors))
    with ck.Checkpoint.open_safetensors(path) as c:
        assert not c.is_mxfp4
        assert (c.config.hidden_dim, c.config.intermediate_dim, c.config.n_experts) == (64, 32, 4)
        data, dtype = c.layer_tensor(2, ck.T_W_MLP2)
        assert dtype == ck.DTYPE_BF16
        assert np.array_equal(data, ckptgen.f32_to_bf16_bits(tensors["block.2.mlp.mlp2_weight"]).ravel())


def test_upload_rejects_bad_arguments_without_a_device(pkg, ck, tmp_path):
    """Every argument check of moe_ckpt_upload_layer comes before the first device call."""
    cfg = ckptgen.TINY
    path = tmp_path / "m.bin"
    ckptgen.write_bin(path, cfg, ckptgen.make_tensors(cfg, seed=8, mxfp4=False))
    with ck.Checkpoint.open_bin(path) as c:
        up = pkg.lib.moe_ckpt_upload_layer
        d = ck.LayerDevice()
        d.struct_bytes = ctypes.sizeof(ck.LayerDevice)
        need = c.staging_bytes()
        assert need == 2 * 32 * 64 * 4 and need % 256 == 0
        fake = 1 << 20  # never dereferenced: each call below fails a check first
        assert up(c._h, 0, ctypes.byref(d), None, need, None) == -1
        assert up(None, 0, ctypes.byref(d), fake, need, None) == -1
        assert up(c._h, 3, ctypes.byref(d), fake, need, None) == -2          # layer out of range
        assert up(c._h, 0, ctypes.byref(d), fake + 16, need, None) == -6     # staging not 256-byte aligned
        assert up(c._h, 0, ctypes.byref(d), fake, need - 1, None) == -4      # staging too small
        d.weight_format = 1
        assert up(c._h, 0, ctypes.byref(d), fake, need, None) == -5          # tiled MXFP4 from a dense file
        d.weight_format = 7
        assert up(c._h, 0, ctypes.byref(d), fake, need, None) == -5
        d.struct_bytes = 12
        assert up(c._h, 0, ctypes.byref(d), fake, need, None) == -5
        # a layer descriptor with every destination NULL uploads nothing and succeeds
        d = ck.LayerDevice()
        d.struct_bytes = ctypes.sizeof(ck.LayerDevice)
        assert up(c._h, 0, ctypes.byref(d), fake, need, None) == 0
