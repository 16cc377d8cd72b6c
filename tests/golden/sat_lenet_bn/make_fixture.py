"""Writes tests/golden/sat_lenet_bn/<set>.npz from the trained parameters N2D2's own DeepNetQAT test loads
(tests/tests_data/mnist_model/weights_8b_SAT and weights_test_SAT, read by tests/Quantizer/QAT/Optimization/
class_DeepNetQAT.cpp:96-103 with LeNet-bn-SAT-8b.ini / LeNet-bn-SAT.ini).  The files are N2D2's text exports: numbers
separated by blanks, one output per line.  Every file becomes one float32 vector under the file's stem, in file order
(convolutions: output, channel, kernel row, kernel column; fully connected: output, input).  Of the `*_quant_weights*`
files (the quantizer's tensor at the last propagate of the training run, one solver step older than the weights beside
it) only those of conv1 and conv2 are kept, as a loose check of the level grid.

    python tests/golden/sat_lenet_bn/make_fixture.py /path/to/N2D2

Only data is read; nothing of N2D2 is imported or run."""
import os
import sys

import numpy as np

SETS = {"weights_8b_SAT": "w8a8", "weights_test_SAT": "w4a4"}


def main(root):
    here = os.path.dirname(os.path.abspath(__file__))
    for folder, name in SETS.items():
        src = os.path.join(root, "tests", "tests_data", "mnist_model", folder)
        arrays = {}
        for f in sorted(os.listdir(src)):
            if f.endswith(".syntxt") and ("quant_weights" not in f or f.startswith(("conv1_", "conv2_"))):
                with open(os.path.join(src, f)) as fh:
                    arrays[f[:-len(".syntxt")]] = np.array(fh.read().split(), dtype=np.float64).astype(np.float32)
        np.savez_compressed(os.path.join(here, name + ".npz"), **arrays)
        print(name, {k: v.size for k, v in arrays.items()})


if __name__ == "__main__":
    main(sys.argv[1])
