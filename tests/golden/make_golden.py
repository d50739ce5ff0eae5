"""Writes tests/golden/*.npz: small input/output vectors for the path.

Run in the build container, where the reference tree is mounted:
    python tests/golden/make_golden.py
Outputs of the P = 1 cases come from the REFERENCE'S OWN csrc/cpu/layernorm.cpp,
compiled from its sources into oracle/_ref/libtw_ref.so (AVX2 configuration,
truncating fp32->bf16 store).  The reference cannot travel to the GPU box; these
vectors can.  The files hold data only (numpy arrays, no pickles):

  ref_fused_add_rms_norm.npz   x, r, w, eps  ->  y_ref, r_ref      per case
  ref_rms_norm.npz             x, w, eps     ->  y_ref             per case

Inputs follow the reference's unit test (tests/kernels/test_layernorm.py:39-44:
x, r ~ N(0,1)/(2H), w ~ N(1, 0.1), seed 0) plus N(0,1) inputs and rows that
exercise the closed forms (constant, one-hot, zero, large magnitude).
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import tw_oracle as O  # noqa: E402

CASES = [  # (name, T, H, eps, input scale)
    ("t7_h8_unit", 7, 8, 1e-6, "test"),
    ("t5_h64_unit", 5, 64, 1e-6, "test"),
    ("t7_h768_unit", 7, 768, 1e-6, "test"),
    ("t3_h5120_unit", 3, 5120, 1e-6, "test"),
    ("t3_h8192_unit", 3, 8192, 1e-6, "test"),
    ("t4_h8192_n01", 4, 8192, 1e-5, "n01"),
    ("t3_h6144_n01", 3, 6144, 1e-5, "n01"),
    ("t6_h256_special", 6, 256, 1e-5, "special"),
]


def draw(rng, T, H, kind):
    w = (1.0 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    if kind == "test":
        s = np.float32(1.0 / (2 * H))
        x = rng.standard_normal((T, H)).astype(np.float32) * s
        r = rng.standard_normal((T, H)).astype(np.float32) * s
    elif kind == "n01":
        x = rng.standard_normal((T, H)).astype(np.float32)
        r = rng.standard_normal((T, H)).astype(np.float32)
    else:  # rows: zero, constant, one-hot, large, tiny, mixed sign cancel
        x = np.zeros((T, H), np.float32)
        r = np.zeros((T, H), np.float32)
        x[1, :] = 1.5; r[1, :] = 0.25
        x[2, 17] = 3.0; r[2, 17] = -1.0
        x[3, :] = 1.0e18 * rng.standard_normal(H); r[3, :] = 1.0e18
        x[4, :] = 1.0e-20 * rng.standard_normal(H)
        x[5, :] = rng.standard_normal(H); r[5, :] = -x[5, :]
    return O.f32_to_bf16(x), O.f32_to_bf16(r), O.f32_to_bf16(w)


def main():
    if not O.have_ref():
        sys.exit("oracle/_ref/libtw_ref.so is missing: run `make -C oracle` where the "
                 "reference tree is mounted")
    rng = np.random.default_rng(0)
    fused, plain = {}, {}
    for name, T, H, eps, kind in CASES:
        x, r, w = draw(rng, T, H, kind)
        y_ref, r_ref = x.copy(), r.copy()
        O.ref_fused_add_rms_norm(y_ref, r_ref, w, eps)
        for k, v in dict(x=x, r=r, w=w, eps=np.float64(eps), y_ref=y_ref, r_ref=r_ref).items():
            fused[f"{name}.{k}"] = v
        o_ref = O.ref_rms_norm(x, w, eps)
        for k, v in dict(x=x, w=w, eps=np.float64(eps), y_ref=o_ref).items():
            plain[f"{name}.{k}"] = v
    np.savez_compressed(os.path.join(HERE, "ref_fused_add_rms_norm.npz"), **fused)
    np.savez_compressed(os.path.join(HERE, "ref_rms_norm.npz"), **plain)
    for f in ("ref_fused_add_rms_norm.npz", "ref_rms_norm.npz"):
        print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
