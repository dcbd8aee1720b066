"""Command-line alias of :mod:`dsv3fp8.convert`, so that
``python convert.py --hf-ckpt-path IN --save-path OUT --n-experts 256 --model-parallel 1`` works from this
directory as it does from the reference's ``inference/`` (convert.py:88-96)."""
from argparse import ArgumentParser

from dsv3fp8.convert import main

if __name__ == "__main__":
    parser = ArgumentParser()
    parser.add_argument("--hf-ckpt-path", type=str, required=True)
    parser.add_argument("--save-path", type=str, required=True)
    parser.add_argument("--n-experts", type=int, required=True)
    parser.add_argument("--model-parallel", type=int, required=True)
    args = parser.parse_args()
    assert args.n_experts % args.model_parallel == 0, "Number of experts must be divisible by model parallelism"
    main(args.hf_ckpt_path, args.save_path, args.n_experts, args.model_parallel)
