"""Paths (same name as src/triton_gated_mlp/const.py:4-6 of the reference)."""

from pathlib import Path

# Directory that holds the package directory's parent: the root of this source tree.
ROOT_PATH = Path(__file__).resolve().parent.parent.parent
