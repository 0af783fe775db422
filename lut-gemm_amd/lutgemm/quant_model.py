"""Quantise the projection layers of a Hugging Face causal language model and write one
packed-weight file per layer: the counterpart of the reference's model walkers
(examples/quant_model_rtn.py:36-113, examples/quant_model_bcq.py:36-97), which only print the
shapes of what they produce.  Same flags; --method selects what the two reference scripts hard-code.

    python -m lutgemm.quant_model --model_name_or_path /path/to/opt --qbits 4 --group_size 128 \\
        --method rtn --out_dir packed/

Each converted layer becomes <out_dir>/<qualified.layer.name>.lutw (readable with
BCQWeight.load / lutgemm_weight_load / `lutgemm_pack info`), its bias, if any, <name>.bias.npy.
Runs on the CPU; nothing is downloaded (the model path must exist locally).
"""
import argparse
import os
import sys

import numpy as np


def parse_args(argv=None):
    ap = argparse.ArgumentParser(description="Quantise a causal language model's projection layers to packed BCQ files")
    ap.add_argument("--model_name_or_path", type=str, required=True, help="local directory of a pretrained model")
    ap.add_argument("--cache_dir", type=str, default=None)
    ap.add_argument("--qbits", type=int, default=4, help="quantisation bits")
    ap.add_argument("--group_size", type=int, default=128, help="weights per scale along the input channels")
    ap.add_argument("--method", choices=["rtn", "bcq"], default="rtn")
    ap.add_argument("--rounds", type=int, default=15, help="alternating refinements (bcq)")
    ap.add_argument("--out_dir", type=str, required=True)
    return ap.parse_args(argv)


def main(argv=None):
    args = parse_args(argv)
    import torch
    from transformers import AutoModelForCausalLM

    import lutgemm
    from lutgemm import quantize

    if not os.path.isdir(args.model_name_or_path):
        sys.exit("quant_model: %s is not a local directory (nothing is downloaded)" % args.model_name_or_path)
    model = AutoModelForCausalLM.from_pretrained(args.model_name_or_path, cache_dir=args.cache_dir,
                                                 local_files_only=True)
    containers = quantize.quantize_model(model, args.qbits, args.group_size, args.method, args.rounds,
                                         to_device=False)
    os.makedirs(args.out_dir, exist_ok=True)
    modules = dict(model.named_modules())
    total_dense = total_packed = 0
    for name, c in containers.items():
        path = os.path.join(args.out_dir, name + ".lutw")
        lutgemm.pack_file(path, c["bW"], c["alpha"], c["k"], c["n"], c["q"], c["num_groups"], c["q_bias"])
        bias = modules[name].bias
        if bias is not None:
            np.save(os.path.join(args.out_dir, name + ".bias.npy"), bias.detach().to(torch.float16).numpy())
        dense, packed = 2 * c["k"] * c["n"], os.path.getsize(path)
        total_dense += dense
        total_packed += packed
        print("%-48s k=%-6d n=%-6d q=%d groups=%-4d %9d B packed (%.2fx smaller than fp16)"
              % (name, c["k"], c["n"], c["q"], c["num_groups"], packed, dense / packed))
    print("%d layers, %.1f MB fp16 -> %.1f MB packed" % (len(containers), total_dense / 1e6, total_packed / 1e6))
    return 0


if __name__ == "__main__":
    sys.exit(main())
