"""Regenerates tests/golden/dlq_inputs.npz: the normal-distributed inputs of DlQuantization's own tests, drawn with
libstdc++'s std::mt19937 / std::normal_distribution<float> exactly as those tests draw them.
Run from the repository root: python tests/golden/make_dlq_inputs.py"""

import os
import subprocess
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    with tempfile.TemporaryDirectory() as tmp:
        exe = os.path.join(tmp, "make_dlq_inputs")
        subprocess.run(["g++", "-O1", "-o", exe, os.path.join(HERE, "make_dlq_inputs.cpp")], check=True)
        out = {}
        for name, mean, std, count in (("normal_mean2_std2", 2, 2, 6000), ("normal_meanm2_std1", -2, 1, 6000),
                                       ("normal_mean2_std2_100k", 2, 2, 100000)):
            path = os.path.join(tmp, name + ".f32")
            subprocess.run([exe, str(mean), str(std), str(count), path], check=True)
            out[name] = np.fromfile(path, dtype=np.float32)
        np.savez_compressed(os.path.join(HERE, "dlq_inputs.npz"), **out)
        for k, v in out.items():
            print(k, v[:4], v.mean(), v.std())


if __name__ == "__main__":
    main()
