"""Writes the on-disk fixtures that pin the checkpoint reader against files the REFERENCE's exporter wrote.

Run in the build container only (it needs /root/reference, which never travels to the GPU box):

    python tests/golden/make_ref_bin.py

It builds a tiny MXFP4 model (tests/ckptgen.py: dense tensors stored as BF16, experts as `.blocks` / `.scales`,
the layout of the published checkpoints), writes it as tests/golden/ref_tiny.safetensors with its config as
tests/golden/ref_tiny_config.json, then imports the reference's
tools/model_export/gpt-oss-20b/export_model_bin.py and runs its main() twice (--dtype float32, --dtype bfloat16)
on those two files.  The exporter's own code reads the safetensors file, dequantises the experts
(dequantize_fp4), orders the tensors (KEYS, CATEGORIES, reorder_keys_for_write) and writes
tests/golden/ref_tiny_f32.bin and tests/golden/ref_tiny_bf16.bin.  Nothing of the exporter is copied: the four
files are data.  tests/test_checkpoint_host.py and tests/test_gpu_checkpoint.py read them.
"""
import importlib.util
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import ckptgen  # noqa: E402

EXPORTER = "/root/reference/tools/model_export/gpt-oss-20b/export_model_bin.py"
CFG = dict(ckptgen.TINY, hidden_size=128, intermediate_size=64, num_experts=8, num_hidden_layers=2)
SEED = 11


def main():
    tensors = ckptgen.make_tensors(CFG, seed=SEED, mxfp4=True)
    st = os.path.join(HERE, "ref_tiny.safetensors")
    cfg_path = os.path.join(HERE, "ref_tiny_config.json")
    dense = [n for n, a in tensors.items() if a.dtype != "uint8"]
    ckptgen.write_safetensors(st, tensors, bf16_names=dense)
    with open(cfg_path, "w") as f:
        json.dump(CFG, f, indent=1, sort_keys=True)
        f.write("\n")
    spec = importlib.util.spec_from_file_location("reference_export_model_bin", EXPORTER)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    for dtype, name in (("float32", "ref_tiny_f32.bin"), ("bfloat16", "ref_tiny_bf16.bin")):
        out = os.path.join(HERE, name)
        sys.argv = [EXPORTER, "--input", st, "--config", cfg_path, "--output", out, "--dtype", dtype]
        mod.main()
        print("wrote %s (%d bytes)" % (out, os.path.getsize(out)))


if __name__ == "__main__":
    main()
