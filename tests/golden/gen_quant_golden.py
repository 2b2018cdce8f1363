"""Writes tests/golden/quant_golden.npz: inputs and the blocks the REFERENCE's own C quantizers produce for them.

Run in the build container only (needs oracle/_ref/ggml_quant_ref, i.e. `make -C oracle ref`, which compiles
third_party/llama.cpp-fork/ggml/src/ggml-quants.c where it lies in the reference tree). The fixture is data:
x [n][32] f32, q8_d [n] u16 (f16 scale bits), q8_q [n][32] i8, q4_blk [n][18] u8 (ggml block_q4_0 bytes), plus the
reference's dequantized values dq8 / dq4 [n][32] f32 for the element reader.
"""
import os
import subprocess
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
TOOL = os.path.join(HERE, "..", "..", "oracle", "_ref", "ggml_quant_ref")


def blocks():
    rng = np.random.Generator(np.random.Philox(20250101))
    out = []
    out.append(rng.standard_normal((1536, 32)).astype(np.float32))                       # plain N(0,1)
    out.append((rng.standard_normal((256, 32)) * 1e-3).astype(np.float32))               # small
    out.append((rng.standard_normal((256, 32)) * 300.0).astype(np.float32))              # large
    out.append((rng.standard_normal((128, 32)) * 1e-7).astype(np.float32))               # scale becomes a subnormal half
    out.append((rng.standard_normal((64, 32)) * 3e-9).astype(np.float32))                # scale rounds to zero in f16
    out.append((rng.standard_normal((64, 32)) * 4e6).astype(np.float32))                 # scale overflows f16
    h = rng.standard_normal((256, 32)).astype(np.float16).astype(np.float32)             # f16-exact inputs
    out.append(h)
    e = np.zeros((40, 32), np.float32)                                                   # closed-form cases
    e[1, 5] = 1.0
    e[2, 5] = -1.0
    e[3, 3], e[3, 9] = 2.0, -2.0          # tie: first (+) wins
    e[4, 3], e[4, 9] = -2.0, 2.0          # tie: first (-) wins
    e[5, :] = 1.0
    e[6, :] = -1.0
    e[7, :] = np.arange(32) - 16          # integers, amax 16 (negative max element)
    e[8, :] = np.arange(32) - 15          # amax 16 positive
    e[9, :] = (np.arange(32) - 15.5) * 0.25
    e[10, 0] = 127.0
    e[10, 1:] = np.arange(31) + 0.5       # x/d lands on k + 0.5 exactly: round half away from zero
    e[11, 0] = -127.0
    e[11, 1:] = -(np.arange(31) + 0.5)
    e[12, 0] = 8.0
    e[12, 1:] = (np.arange(31) % 16) - 7.5   # q4: x*id + 8.5 lands on integers / halves
    e[13, 0] = -8.0
    e[13, 1:] = (np.arange(31) % 16) - 7.5
    e[14, 31] = 3.5                       # max at the last index
    e[15, :] = np.float32(1e-45)          # f32 denormal everywhere
    e[16, 0], e[16, 1] = 1.0, np.float32(1.0) - np.float32(2.0 ** -24)
    e[17, 0], e[17, 16] = 5.0, -5.0       # tie across the nibble halves
    e[18, 16], e[18, 0] = 5.0, -5.0
    for i in range(19, 40):               # random sign/tie patterns on a coarse grid
        e[i] = rng.integers(-4, 5, 32).astype(np.float32) * np.float32(0.5 ** (i - 19))
    out.append(e)
    g = rng.integers(-8, 9, (128, 32)).astype(np.float32) * 0.125                        # many ties
    out.append(g)
    return np.concatenate(out, 0)


def run(mode, data):
    with tempfile.TemporaryDirectory() as d:
        fi, fo = os.path.join(d, "in.bin"), os.path.join(d, "out.bin")
        data.tofile(fi)
        subprocess.run([TOOL, mode, fi, fo], check=True)
        return np.fromfile(fo, dtype=np.uint8)


def main():
    x = blocks()
    n = x.shape[0]
    b8 = run("q8_0", x).reshape(n, 34)
    b4 = run("q4_0", x).reshape(n, 18)
    dq8 = run("dq8_0", b8).view(np.float32).reshape(n, 32)
    dq4 = run("dq4_0", b4).view(np.float32).reshape(n, 32)
    np.savez_compressed(
        os.path.join(HERE, "quant_golden.npz"), x=x,
        q8_d=b8[:, :2].copy().view(np.uint16).reshape(n), q8_q=b8[:, 2:].copy().view(np.int8),
        q4_blk=b4, dq8=dq8, dq4=dq4)
    print("wrote", n, "blocks")


if __name__ == "__main__":
    main()
