"""Writes the data fixtures of this directory.  Run in the development container, where the
reference checkout is mounted; the GPU box only sees the files written here.

deeplandmark_2_LE1.caffemodel
    The trained parameters (binary NetParameter, 70 KB) of the level-2 left-eye landmark
    net that ships with the reference as example data
    (example/models/deeplandmark/2_LE1.caffemodel): one of the few files in its tree with
    real trained weights.  It is copied byte for byte; the tests build the matching net
    definition themselves (tests/test_nets_gpu.py) and compare the HIP forward pass on these
    weights with the CPU oracle.
"""
import os
import shutil
import sys

REF = os.environ.get("MINICAFFE_REFERENCE", "/root/reference")
HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    src = os.path.join(REF, "example", "models", "deeplandmark", "2_LE1.caffemodel")
    if not os.path.exists(src):
        sys.exit("reference checkout not found at %s" % REF)
    dst = os.path.join(HERE, "deeplandmark_2_LE1.caffemodel")
    shutil.copyfile(src, dst)
    print("wrote %s (%d bytes)" % (dst, os.path.getsize(dst)))


if __name__ == "__main__":
    main()
