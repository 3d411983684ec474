"""GPU tests of the checkpoint reader: a file in either on-disk format, uploaded through
moe_ckpt_upload_layer, must give the block the same weights bit for bit, and the block's output
must match the CPU oracle run on the weights the test wrote."""
import os

import numpy as np
import pytest
import torch

import ckptgen
import hostgen

pytestmark = pytest.mark.gpu

OUT_TOL = 1e-2  # max|y - ref| / max|ref|

CFG = dict(ckptgen.TINY, hidden_size=128, intermediate_size=64, num_experts=8, num_hidden_layers=2)


@pytest.fixture(scope="module")
def ck(pkg):
    import importlib
    return importlib.import_module("gpt_oss_amd_amd.checkpoint")


def bits_of(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def oracle_layer(oracle, tensors, layer, x, K, mxfp4):
    p = "block.%d.mlp." % layer
    if mxfp4:
        w1 = ckptgen.mxfp4_dequant(tensors[p + "mlp1_weight.blocks"], tensors[p + "mlp1_weight.scales"])
        w2 = ckptgen.mxfp4_dequant(tensors[p + "mlp2_weight.blocks"], tensors[p + "mlp2_weight.scales"])
    else:
        w1, w2 = tensors[p + "mlp1_weight"], tensors[p + "mlp2_weight"]
    return oracle.moe_block(x, tensors[p + "gate.weight"], tensors[p + "gate.bias"], w1, tensors[p + "mlp1_bias"], w2,
                            tensors[p + "mlp2_bias"], K, 7.0, want_scores=True), (w1, w2)


@pytest.mark.parametrize("bf16_payload", [False, True])
def test_bin_to_block(pkg, ck, oracle, dev, tmp_path, bf16_payload):
    tensors = ckptgen.make_tensors(CFG, seed=11, mxfp4=False)
    path = tmp_path / "model.bin"
    ckptgen.write_bin(path, CFG, tensors, bf16=bf16_payload)
    rng = np.random.default_rng(1)
    x = rng.standard_normal((37, 128)).astype(np.float32)
    with ck.Checkpoint.open_bin(path, ck.DTYPE_BF16 if bf16_payload else ck.DTYPE_F32) as c:
        for layer in (0, 1):
            print("bin layer", layer, "bf16 payload", bf16_payload, flush=True)
            # smallest legal staging buffer: the expert tensors go through it in several pieces
            staging = torch.empty(c.staging_bytes(), dtype=torch.uint8, device=dev)
            t = c.upload_layer(layer, device=dev, staging=staging)
            p = "block.%d.mlp." % layer
            for key, name in (("w_router", "gate.weight"), ("b_router", "gate.bias"), ("w_mlp1", "mlp1_weight"),
                              ("b_mlp1", "mlp1_bias"), ("w_mlp2", "mlp2_weight"), ("b_mlp2", "mlp2_bias"),
                              ("rms_ffn_w", "norm.scale")):
                assert np.array_equal(bits_of(t[key]).ravel(), ckptgen.f32_to_bf16_bits(tensors[p + name]).ravel()), key
            blk = c.moe_block(layer, max_tokens=64, device=dev)
            y, ti, tv = blk.forward(torch.from_numpy(x).to(dev))
            torch.cuda.synchronize()
            (ref_y, ref_i, ref_v, _), _ = oracle_layer(oracle, tensors, layer, x, CFG["experts_per_token"], False)
            assert np.array_equal(ti.cpu().numpy(), ref_i)
            assert np.allclose(tv.cpu().numpy(), ref_v, rtol=1e-6, atol=1e-7)
            assert hostgen.rel_err(y.cpu().numpy(), ref_y) <= OUT_TOL


@pytest.mark.parametrize("tiled", [True, False])
def test_safetensors_mxfp4_to_block(pkg, ck, oracle, dev, tmp_path, tiled):
    tensors = ckptgen.make_tensors(CFG, seed=12, mxfp4=True)
    bf16_names = {n for n in tensors if n.endswith("bias") or n.endswith("gate.weight") or n.endswith("norm.scale")}
    path = tmp_path / "model.safetensors"
    ckptgen.write_safetensors(path, tensors, bf16_names, metadata={"format": "pt"})
    want = ck.CkptConfig()
    want.experts_per_token, want.swiglu_limit = CFG["experts_per_token"], CFG["swiglu_limit"]
    rng = np.random.default_rng(2)
    x = rng.standard_normal((50, 128)).astype(np.float32)
    E, H, I = 8, 128, 64
    with ck.Checkpoint.open_safetensors(path, want) as c:
        assert c.is_mxfp4
        for layer in (0, 1):
            print("safetensors layer", layer, "tiled", tiled, flush=True)
            staging = torch.empty(c.staging_bytes(), dtype=torch.uint8, device=dev)
            t = c.upload_layer(layer, device=dev, tiled=tiled, staging=staging)
            p = "block.%d.mlp." % layer
            want1 = oracle.dequant_mxfp4(tensors[p + "mlp1_weight.blocks"], tensors[p + "mlp1_weight.scales"])
            want2 = oracle.dequant_mxfp4(tensors[p + "mlp2_weight.blocks"], tensors[p + "mlp2_weight.scales"])
            if tiled:
                got1 = bits_of(pkg.mxfp4_tiled_to_bf16(t["w_mlp1"], t["w_mlp1_scales"], E, 2 * I, H))
                got2 = bits_of(pkg.mxfp4_tiled_to_bf16(t["w_mlp2"], t["w_mlp2_scales"], E, H, I))
            else:
                got1, got2 = bits_of(t["w_mlp1"]), bits_of(t["w_mlp2"])
            assert np.array_equal(got1.ravel(), want1.ravel()) and np.array_equal(got2.ravel(), want2.ravel())
            assert np.array_equal(bits_of(t["b_mlp2"]).ravel(), ckptgen.f32_to_bf16_bits(tensors[p + "mlp2_bias"]).ravel())
            blk = c.moe_block(layer, max_tokens=64, device=dev, tiled=tiled)
            y, ti, tv = blk.forward(torch.from_numpy(x).to(dev))
            torch.cuda.synchronize()
            (ref_y, ref_i, ref_v, _), (w1, w2) = oracle_layer(oracle, tensors, layer, x, CFG["experts_per_token"], True)
            # the test-side dequantiser agrees with the oracle's, so the reference output is built
            # from the same weights the device holds
            assert np.array_equal(ckptgen.f32_to_bf16_bits(w1).ravel(), want1.ravel())
            assert np.array_equal(ti.cpu().numpy(), ref_i)
            assert hostgen.rel_err(y.cpu().numpy(), ref_y) <= OUT_TOL


def test_upload_rejects_bad_arguments(pkg, ck, dev, tmp_path):
    import ctypes
    tensors = ckptgen.make_tensors(CFG, seed=13, mxfp4=False)
    path = tmp_path / "model.bin"
    ckptgen.write_bin(path, CFG, tensors)
    with ck.Checkpoint.open_bin(path) as c:
        small = torch.empty(256, dtype=torch.uint8, device=dev)
        with pytest.raises(Exception) as e:
            c.upload_layer(0, device=dev, staging=small)
        assert e.value.code == -4
        with pytest.raises(Exception) as e:
            c.upload_layer(0, device=dev, tiled=True)     # dense file cannot give tiled MXFP4
        assert e.value.code == -5
        with pytest.raises(Exception) as e:
            c.upload_layer(2, device=dev)
        assert e.value.code == -2
        d = ck.LayerDevice()
        d.struct_bytes = 8
        st = torch.empty(c.staging_bytes(), dtype=torch.uint8, device=dev)
        assert pkg.lib.moe_ckpt_upload_layer(c._h, 0, ctypes.byref(d), st.data_ptr(), st.numel(), None) == -5


GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_reference_written_files_to_block(pkg, ck, oracle, dev):
    """The files under tests/golden/ that the reference's export_model_bin.py read (ref_tiny.safetensors) and wrote
    (ref_tiny_f32.bin, ref_tiny_bf16.bin, through its own dequantize_fp4): uploaded through the three routes
    (.bin fp32, .bin bf16, safetensors dequantised on the device) every MoE tensor must come out as the same BF16
    bits, and the three blocks must give the same output as the oracle on those weights."""
    assert CFG == dict(ckptgen.TINY, hidden_size=128, intermediate_size=64, num_experts=8, num_hidden_layers=2)
    tensors = ckptgen.make_tensors(CFG, seed=11, mxfp4=True)
    want = ck.CkptConfig()
    want.experts_per_token, want.swiglu_limit = CFG["experts_per_token"], CFG["swiglu_limit"]
    rng = np.random.default_rng(3)
    x = rng.standard_normal((41, 128)).astype(np.float32)
    keys = ("w_router", "b_router", "w_mlp1", "b_mlp1", "w_mlp2", "b_mlp2", "rms_ffn_w")
    with ck.Checkpoint.open_bin(os.path.join(GOLDEN, "ref_tiny_f32.bin"), ck.DTYPE_F32) as c32, \
            ck.Checkpoint.open_bin(os.path.join(GOLDEN, "ref_tiny_bf16.bin"), ck.DTYPE_BF16) as c16, \
            ck.Checkpoint.open_safetensors(os.path.join(GOLDEN, "ref_tiny.safetensors"), want) as cst:
        for layer in (0, 1):
            print("reference-written files, layer", layer, flush=True)
            p = "block.%d.mlp." % layer
            t32 = c32.upload_layer(layer, device=dev)
            t16 = c16.upload_layer(layer, device=dev)
            tst = cst.upload_layer(layer, device=dev, tiled=False)
            for key in keys:
                a, b, s = bits_of(t32[key]).ravel(), bits_of(t16[key]).ravel(), bits_of(tst[key]).ravel()
                assert np.array_equal(a, b), key
                assert np.array_equal(a, s), key  # device dequantiser == the reference's dequantize_fp4
            assert np.array_equal(bits_of(t32["w_mlp1"]).ravel(),
                                  oracle.dequant_mxfp4(tensors[p + "mlp1_weight.blocks"],
                                                       tensors[p + "mlp1_weight.scales"]).ravel())
            (ref_y, ref_i, ref_v, _), _ = oracle_layer(oracle, tensors, layer, x, CFG["experts_per_token"], True)
            for name, c, kw in (("bin f32", c32, {}), ("bin bf16", c16, {}), ("safetensors tiled", cst, {"tiled": True})):
                blk = c.moe_block(layer, max_tokens=64, device=dev, **kw)
                y, ti, tv = blk.forward(torch.from_numpy(x).to(dev))
                torch.cuda.synchronize()
                assert np.array_equal(ti.cpu().numpy(), ref_i), name
                err = hostgen.rel_err(y.cpu().numpy(), ref_y)
                print("  %s: max-rel %.3g rms-rel %.3g" % (name, err, hostgen.rms_err(y.cpu().numpy(), ref_y)), flush=True)
                assert err <= OUT_TOL, name
