#!/usr/bin/env python3
"""Writes tests/golden/mxfp4_golden.npz from the reference's own MX element math.

Runs only where the reference tree is mounted: it needs oracle/_ref/libmxref.so,
the shared object that `make -C oracle ref` compiles from the reference's
src/csrc/mxfp_quant.h (a dependency-free C++ header).  The vectors are

  e2m1_bf16_out  quantize_elemwise(v, 3, 2, 6.0, rd_even, true, true) for every
                 one of the 65536 bf16 bit patterns v (as fp32 bits)
  tie_in/out     the same for fp32 values at and next to every rounding
                 boundary of the E2M1 grid, both signs, and random fp32 values
  scale_bf16_out mx_get_shared_scale(biased_exp(a), 8, 6.0) for every
                 non-negative bf16 bit pattern a (fp32 bits of the scale)
  scale_in/out   the same for random positive fp32 values incl. subnormals
"""
import ctypes
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
REF = os.path.join(ROOT, "oracle", "_ref", "libmxref.so")


def main():
    R = ctypes.CDLL(REF)
    vp, cl = ctypes.c_void_p, ctypes.c_long
    R.ref_e2m1_round_n.argtypes = [vp, vp, cl]
    R.ref_mx_shared_scale_n.argtypes = [vp, vp, cl]

    def e2m1(a):
        a = np.ascontiguousarray(a, np.float32)
        o = np.empty_like(a)
        R.ref_e2m1_round_n(a.ctypes.data, o.ctypes.data, a.size)
        return o

    def scale(a):
        a = np.ascontiguousarray(a, np.float32)
        o = np.empty_like(a)
        R.ref_mx_shared_scale_n(a.ctypes.data, o.ctypes.data, a.size)
        return o

    bf16_all = (np.arange(65536, dtype=np.uint32) << 16).view(np.float32)
    rng = np.random.default_rng(20240607)
    ties = np.array([0.25, 0.5, 0.75, 1.0, 1.25, 1.5, 1.75, 2.0, 2.5, 3.0, 3.5, 4.0, 5.0, 6.0, 7.0, 8.0], np.float32)
    near = []
    for t in ties:
        b = int(np.float32(t).view(np.uint32))
        for d in range(-3, 4):
            near.append(np.array([b + d], np.uint32).view(np.float32)[0])
    near = np.array(near, np.float32)
    rnd = (rng.standard_normal(20000) * 3).astype(np.float32)
    tiny = (rng.standard_normal(2000) * 1e-3).astype(np.float32)
    tie_in = np.concatenate([near, -near, rnd, tiny])
    sc_rand = np.abs(rng.standard_normal(4000).astype(np.float32)) * np.float32(10.0) ** rng.integers(-44, 38, 4000).astype(np.float32)
    sc_rand = sc_rand.astype(np.float32)
    out = {
        "e2m1_bf16_out": e2m1(bf16_all).view(np.uint32),
        "tie_in": tie_in.view(np.uint32),
        "tie_out": e2m1(tie_in).view(np.uint32),
        "scale_bf16_out": scale(bf16_all[:32768]).view(np.uint32),
        "scale_in": sc_rand.view(np.uint32),
        "scale_out": scale(sc_rand).view(np.uint32),
    }
    np.savez_compressed(os.path.join(HERE, "mxfp4_golden.npz"), **out)
    print({k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
