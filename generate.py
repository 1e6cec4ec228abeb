#!/usr/bin/env python3
"""python generate.py --model DIR | --random PRESET [options]: see ``simple-inference_amd/cli.py``."""

import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

from simple_inference_amd.cli import main  # noqa: E402

if __name__ == "__main__":
    sys.exit(main())
