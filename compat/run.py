"""Run one of the reference's scripts against the MI355X operators, unedited:

    python /path/to/this/repo/compat/run.py train.py --attn_type 24 ...

is ``python train.py --attn_type 24 ...`` with this directory ahead of the script's own on
``sys.path``, so that ``from utils.fast_fast_weight import fast_weight_delta`` and its like
(language_modeling/src/utils/cuda_fast_weight_layer.py:9-23, algorithmic/layers.py:7-10,
reinforcement_learning/torchbeast/layer.py:7-10) find the shim modules here instead of the
reference's CUDA extensions.
"""
import os
import runpy
import sys


def main():
    if len(sys.argv) < 2:
        sys.exit("usage: python compat/run.py script.py [args ...]")
    here = os.path.dirname(os.path.abspath(__file__))
    script = os.path.abspath(sys.argv[1])
    sys.argv = sys.argv[1:]
    sys.path[0] = os.path.dirname(script)      # what `python script.py` would have put there
    sys.path.insert(0, here)
    runpy.run_path(script, run_name="__main__")


if __name__ == "__main__":
    main()
