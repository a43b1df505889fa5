#!/usr/bin/env python3
"""Writes tests/golden/ref_vectors.npz: inputs and the outputs the reference's own CPU MoE header
(src/qwen38_cpu_moe.cuh, compiled as oracle/_ref/libwdref.so by oracle/Makefile) produces for them.

Run in a container that has the reference tree mounted:  python tests/golden/make_fixtures.py
The file holds data only (numpy arrays); tests/test_golden.py checks the CPU oracle and the HIP library
against it where the reference itself is absent.
"""
import ctypes as C
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import pyoracle as po          # noqa: E402
from warpdecode_amd import synth           # noqa: E402

SEED = synth.BASE_SEED
TYPES = [("iq3_s", synth.IQ3_S), ("iq2_s", synth.IQ2_S), ("iq4_nl", synth.IQ4_NL), ("q8_0", synth.Q8_0)]
COLS = [256, 512, 2048, 2560]
MAKERS = {synth.IQ3_S: synth.iq3_s_matrix, synth.IQ2_S: synth.iq2_s_matrix, synth.IQ4_NL: synth.iq4_nl_matrix,
          synth.Q8_0: synth.q8_0_matrix}


def main():
    r = po.ref()
    if r is None:
        sys.exit("oracle/_ref/libwdref.so is not built (needs /root/reference): make -C oracle all")
    f32p, i8p, u16p, i16p = (C.POINTER(t) for t in (C.c_float, C.c_int8, C.c_uint16, C.c_int16))
    out = {}

    # activations: unit-rms noise with a zero block, a tiny block (fp16 scale below 2^-24), a huge block
    for cols in COLS:
        rng = synth.rng_for(SEED, 7000 + cols)
        x = synth.rms_normed(rng, cols)
        x[32:64] = 0.0
        if cols >= 512:
            x[64:96] *= np.float32(1e-7)
            x[256:288] *= np.float32(3e4)
        out["x_%d" % cols] = x
        qs, d = np.empty(cols, np.int8), np.empty(cols // 32, np.uint16)
        r.wdref_quantize_q8_0(x.ctypes.data_as(f32p), cols, qs.ctypes.data_as(i8p), d.ctypes.data_as(u16p))
        out["q8_0_qs_%d" % cols], out["q8_0_d_%d" % cols] = qs, d
        kq, kd, kb = np.empty(cols, np.int8), np.empty(cols // 256, np.float32), np.empty(cols // 16, np.int16)
        r.wdref_quantize_q8_K(x.ctypes.data_as(f32p), cols, kq.ctypes.data_as(i8p), kd.ctypes.data_as(f32p),
                              kb.ctypes.data_as(i16p))
        out["q8_k_qs_%d" % cols], out["q8_k_d_%d" % cols], out["q8_k_bsums_%d" % cols] = kq, kd, kb
        # weight rows of every type against that activation: AVX2-order and scalar-order results
        for name, t in TYPES:
            rng_w = synth.rng_for(SEED, 7100 + cols, t)
            w = MAKERS[t](rng_w, 4, cols)
            aq, ad = (kq, kd) if t in (synth.IQ3_S, synth.IQ2_S) else (qs, d)
            out["w_%s_%d" % (name, cols)] = w
            out["y_%s_%d" % (name, cols)] = np.array([po.ref_row(t, w[i], cols, aq, ad) for i in range(4)], np.float32)
            out["y_scalar_%s_%d" % (name, cols)] = np.array([po.ref_row(t, w[i], cols, aq, ad, scalar=True)
                                                             for i in range(4)], np.float32)

    # transcendental helpers on a spread of arguments incl. the overflow / underflow branches
    rng = synth.rng_for(SEED, 7200)
    v = np.concatenate([rng.standard_normal(192).astype(np.float32) * 8, np.float32([0, -0.0, 88.5, -88.5, 130, -130, 200,
                        -200, 1e-30, -1e-30, 17.25, -103.9])]).astype(np.float32)
    out["fn_x"] = v
    out["fn_exp"] = np.array([r.wdref_exp(float(a)) for a in v], np.float32)
    out["fn_silu"] = np.array([r.wdref_silu(float(a)) for a in v], np.float32)
    out["fn_sigmoid"] = np.array([r.wdref_sigmoid(float(a)) for a in v], np.float32)

    # F32 dot in the 4x8 accumulator order, ragged lengths included
    for n in (8, 31, 32, 100, 2048):
        a, b = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
        out["dot_a_%d" % n], out["dot_b_%d" % n] = a, b
        out["dot_y_%d" % n] = np.float32(r.wdref_dot_f32(a.ctypes.data_as(f32p), b.ctypes.data_as(f32p), n))

    # a tiny routed layer through run_layer (ids and weights given) and the shared-expert Q8_0 chain
    H, F, E, k = 256, 64, 4, 2
    L = synth.make_layer(H, F, E, k, synth.IQ3_S, synth.Q8_0, shared=True, layer=70)
    x = synth.rms_normed(synth.rng_for(SEED, 7300), H)
    ids, wts = np.int32([2, 0]), np.float32([0.625, 0.375])
    out["layer_x"], out["layer_ids"], out["layer_weights"] = x, ids, wts
    for name in ("gate", "up", "down", "shared_gate", "shared_up", "shared_down"):
        out["layer_" + name] = np.ascontiguousarray(L[name])
    out["layer_routed"] = po.ref_run_layer(L, x, ids, wts, threads=1)
    out["layer_shared"] = po.ref_q8_0_chain(L["shared_gate"], L["shared_up"], L["shared_down"], H, F, x)
    out["layer_geometry"] = np.int32([H, F, E, k])

    path = os.path.join(ROOT, "tests", "golden", "ref_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote %s: %d arrays, %d bytes" % (path, len(out), os.path.getsize(path)))


if __name__ == "__main__":
    main()
