"""Writes tests/golden/q8_golden.npz: small seeded inputs with the CPU
oracle's outputs, so that the GPU path and later oracle builds are checked
against committed data rather than against whatever the generators produce
on the day. Run from the repository root:  python tests/golden/make_golden.py

The reference is Rust and cannot be built or run here, so these vectors come
from the C restatement (oracle/q8_oracle.c) after it passed its pinning
tests; the entries under "known_*" are the reference's own known answers,
typed in from its test modules (file:line in the key comments below).
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle as O  # noqa: E402
from tuckmill_amd import synth as S  # noqa: E402

out = {}

# crates/tuckcore/src/tensor.rs:264-272 and :358-370
out["known_f16_bits"] = np.array([0x3C00, 0xC000, 0x0000, 0x0001], np.uint16)
out["known_f16_values"] = np.array([1.0, -2.0, 0.0, 2.0 ** -24], np.float32)
out["known_f32_inputs"] = np.array([0.0, 1.0, -2.0, 65504.0, 100000.0, 5.96e-8,
                                    1.0 + 2.0 ** -11, 1.0 + 2.0 ** -11 + 2.0 ** -13], np.float32)
out["known_f32_to_f16"] = np.array([0x0000, 0x3C00, 0xC000, 0x7BFF, 0x7C00, 0x0001, 0x3C00, 0x3C01],
                                   np.uint16)
# crates/tuckcore/src/tensor.rs:373-392
xq = np.zeros(32, np.float32)
xq[0], xq[1], xq[2] = 127.0, -63.5, 1.0
out["known_quant_x"] = xq
out["known_quant_q"] = np.array([127, -64, 1] + [0] * 29, np.int8)
out["known_quant_d"] = np.array([1.0], np.float32)

# xorshift64* streams of the reference's tests (crates/metal/src/tests.rs:30-40)
for seed in (1, 3, 5, 7, 11, 13):
    r = O.Rng(seed)
    out[f"rng_{seed}"] = np.array([r.next() for _ in range(64)], np.uint64)
out["boundary_weights_17_64_3"] = O.boundary_weights(17, 64, 3)
out["boundary_input_64_3"] = O.boundary_input(64, 3 ^ 0x9E37)

# seeded products: (rows, cols, batch)
for i, (rows, cols, batch) in enumerate([(48, 1024, 1), (33, 1152, 4), (20, 96, 3), (64, 2048, 2)]):
    w = S.make_weights(rows, cols, 900 + i, threads=1)
    x = S.make_activations(cols * batch, 900 + i)
    out[f"case{i}_dims"] = np.array([rows, cols, batch], np.int64)
    out[f"case{i}_w"] = w
    out[f"case{i}_x"] = x
    out[f"case{i}_y_f32"] = O.gemm_q8_0_f32(w, rows, cols, x, batch)
    out[f"case{i}_y_q8"] = O.gemm_q8_0_q8_0(w, rows, cols, x, batch)
    qs, ds = O.quantize_row_q8_0(x)
    out[f"case{i}_xq"] = qs
    out[f"case{i}_xd"] = ds
# boundary data through both CPU orders
w = O.boundary_weights(17, 64, 3)
x = O.boundary_input(64, 3 ^ 0x9E37)
out["boundary_y_kernels_order"] = O.gemv_q8_0_f32(w, 17, 64, x)
out["boundary_y_dequant_first"] = O.gemv_q8_0_f32_dequant_first(w, 17, 64, x)

path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "q8_golden.npz")
np.savez_compressed(path, **out)
print("wrote", path, os.path.getsize(path), "bytes")
