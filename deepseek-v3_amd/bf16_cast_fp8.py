"""Command-line alias of :mod:`dsv3fp8.bf16_cast_fp8`:
``python bf16_cast_fp8.py --input-bf16-hf-path IN --output-fp8-hf-path OUT`` -- the inverse of
``fp8_cast_bf16.py`` beside it (reference: inference/fp8_cast_bf16.py:106-111 for the command-line shape)."""
from argparse import ArgumentParser

from dsv3fp8.bf16_cast_fp8 import main

if __name__ == "__main__":
    parser = ArgumentParser()
    parser.add_argument("--input-bf16-hf-path", type=str, required=True)
    parser.add_argument("--output-fp8-hf-path", type=str, required=True)
    parser.add_argument("--scale-fmt", type=str, default=None, choices=[None, "ue8m0"])
    args = parser.parse_args()
    main(args.input_bf16_hf_path, args.output_fp8_hf_path, scale_fmt=args.scale_fmt)
