#!/usr/bin/env python3
"""Greedy generation with a Narurax checkpoint (config.json + model.safetensors) on the ragged stack engine:

    python run.py --model_dir DIR --input_tokens prompt.csv|prompt.npy --max_output_len 32 [--dtype bfloat16|float32]

The model class is chosen by config.json through the model registry, so this is the command line of examples/tolenex/run.py
(same arguments, same outputs): ids in, ids out, several prompts run as one continuously batched job."""
import os
import sys

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), '..', 'tolenex'))

from run import generate, parse_arguments  # noqa: E402

if __name__ == '__main__':
    generate(**vars(parse_arguments()))
