"""Random-weights mode on the command line: writes a model folder (config.json and
model.safetensors) from a configuration and a seed.

    python -m mini_llm_amd.cli.random_model --config config.json --seed 5 --out DIR [--dtype bfloat16]"""

from __future__ import annotations

import argparse
import json
import sys


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(description="Write a model folder with random weights")
    parser.add_argument("--config", required=True, help="a config.json of a registered architecture")
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--out", required=True)
    parser.add_argument("--dtype", default="float32", choices=("float32", "bfloat16"), help="element type stored in the file")
    args = parser.parse_args(argv)
    from ..config import config_from_dict
    from ..weights import write_model_dir

    with open(args.config) as f:
        config = config_from_dict(json.load(f))
    print(write_model_dir(config, args.seed, args.out, args.dtype))
    return 0


if __name__ == "__main__":
    sys.exit(main())
