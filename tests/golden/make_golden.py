"""Writes the small golden fixtures of tests/golden/ from the CPU oracle.

Nothing here comes from running the reference (it is Rust and cannot be built in this environment):
literal_blocks.npz holds the three hand-written blocks of the reference's unit tests
(crates/strix-models/src/ggml_quant.rs:443-469, 497-514) with the outputs those tests assert;
the q*_small.npz cases are seeded synthetic tensors with the oracle's i32 block dots and fp32 outputs.

    python tests/golden/make_golden.py
"""
import importlib.util
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))


def load(name, path):
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


orc = load("strix_oracle", os.path.join(ROOT, "oracle", "strix_oracle.py"))
synth = load("strix_rs_amd_synth", os.path.join(ROOT, "strix.rs_amd", "synth.py"))


def f16b(v):
    h = orc.f32_to_f16(v)
    return [h & 0xff, h >> 8]


def literal_blocks():
    q8 = np.array(f16b(0.5) + [(i - 4) & 0xff for i in range(32)], np.uint8)
    q8_out = (0.5 * (np.arange(32) - 4.0)).astype(np.float32)            # ggml_quant.rs:450-452
    qs = [0] * 16
    qs[0], qs[1] = 0x80, 0xF1
    q4 = np.array(f16b(2.0) + qs, np.uint8)
    q4_out = np.full(32, -16.0, np.float32)                               # nibble 0 -> (0-8)*2
    q4_out[0], q4_out[16], q4_out[1], q4_out[17] = -16.0, 0.0, -14.0, 14.0  # ggml_quant.rs:465-468
    q6 = np.zeros(210, np.uint8)
    q6[0], q6[128] = 0x05, 0x01
    q6[192:208] = 1
    q6[208:210] = f16b(1.0)
    q6_out = np.full(256, -32.0, np.float32)                              # ggml_quant.rs:511-512
    q6_out[0] = -11.0                                                     # ggml_quant.rs:509
    np.savez(os.path.join(HERE, "literal_blocks.npz"), q8_0_raw=q8, q8_0_out=q8_out, q4_0_raw=q4,
             q4_0_out=q4_out, q6_k_raw=q6, q6_k_out=q6_out)


def small_case(name, ty, N, K, m, seed):
    raw = synth.make_weight(ty, N, K, seed)
    x = synth.make_acts(m, K, seed + 1)
    xq, xd, xs = orc.actquant(x, K)
    dots = np.stack([orc.block_dots(ty, raw, K, N, xq[t]) for t in range(m)])
    y = orc.matmul_q8(ty, raw, K, N, xq, xd)
    yf = orc.matmul_f32(ty, raw, K, N, x, 1)
    np.savez(os.path.join(HERE, name), ty=ty, N=N, K=K, raw=raw, x=x, xq=xq, xd=xd, xs16=xs,
             block_dots=dots, y_q8=y, y_f32=yf)


if __name__ == "__main__":
    literal_blocks()
    small_case("q4_0_small.npz", 2, 8, 64, 2, 1001)
    small_case("q8_0_small.npz", 8, 8, 64, 2, 1002)
    small_case("q6_k_small.npz", 14, 4, 256, 1, 1003)
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
