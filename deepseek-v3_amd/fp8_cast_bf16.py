"""Command-line alias of :mod:`dsv3fp8.fp8_cast_bf16`, so that
``python fp8_cast_bf16.py --input-fp8-hf-path IN --output-bf16-hf-path OUT`` works from this directory as it
does from the reference's ``inference/`` (fp8_cast_bf16.py:106-111)."""
from argparse import ArgumentParser

from dsv3fp8.fp8_cast_bf16 import main

if __name__ == "__main__":
    parser = ArgumentParser()
    parser.add_argument("--input-fp8-hf-path", type=str, required=True)
    parser.add_argument("--output-bf16-hf-path", type=str, required=True)
    args = parser.parse_args()
    main(args.input_fp8_hf_path, args.output_bf16_hf_path)
