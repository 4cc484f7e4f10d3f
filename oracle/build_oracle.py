"""Compile the oracle's C sources (gcc) into oracle/_build/ -- test infrastructure."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
OUT_DIR = os.path.join(HERE, "_build")
LIB = os.path.join(OUT_DIR, "libconv_direct.so")


def build():
    os.makedirs(OUT_DIR, exist_ok=True)
    src = os.path.join(HERE, "conv_direct.c")
    subprocess.run(["gcc", "-O2", "-std=c99", "-fPIC", "-shared", "-o", LIB, src], check=True)
    return LIB


if __name__ == "__main__":
    print("built", build())
