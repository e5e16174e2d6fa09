"""Writes tests/golden/vectors.npz: small seeded inputs of every operation of the path with the
outputs the CPU oracle gives for them, so that a parity failure can be told from an oracle change
(the CPU suite checks the oracle still reproduces them) and the GPU suite has committed vectors to
meet. Run from the repository root: python tests/golden/make_fixtures.py"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402
from llmp_amd import synth  # noqa: E402


def build():
    out = {}
    # llmp.q8_1: 3 rows of 320 values (one block all zero, one with a lone huge value).
    x = synth.activations(3, 320, 11)
    x[1, 32:64] = 0.0
    x[2, 5] = 1.0e4
    out["q8_x"] = x
    out["q8_blocks"] = oracle.q8_1_quantize(x)
    # llmp.vecq, Q8_0, dense, 2 tokens.
    k, n = 256, 24
    w8 = synth.q8_0_weights(n, k, 12)
    a = synth.activations(2, k, 13)
    q8 = oracle.q8_1_quantize(a)
    out["q8_0_w"], out["q8_0_x"] = w8, a
    out["q8_0_y"] = oracle.vecq(oracle.TYPE_Q8_0, w8, q8, k, n, tokens=2)
    out["q8_0_sums"] = oracle.vecq_block_sums(oracle.TYPE_Q8_0, w8, q8[:1], k, n)
    # llmp.vecq, Q4_K, gate/up with each GLU, 1 token, and the block sums.
    k, n = 512, 20
    up, gate = synth.q4_k_weights(n, k, 14), synth.q4_k_weights(n, k, 15)
    a = synth.activations(1, k, 16)
    q8 = oracle.q8_1_quantize(a)
    out["q4_k_up"], out["q4_k_gate"], out["q4_k_x"] = up, gate, a
    out["q4_k_y"] = oracle.vecq(oracle.TYPE_Q4_K, up, q8, k, n)
    for kind in (1, 2, 3):
        out[f"q4_k_glu{kind}"] = oracle.vecq(oracle.TYPE_Q4_K, up, q8, k, n, gate=gate, glu=kind, limit=0.05 if kind == 2 else 0.0)
    out["q4_k_sums"] = oracle.vecq_block_sums(oracle.TYPE_Q4_K, up, q8, k, n)
    # llmp.vecq, Q4_0 (the legacy block that reads the activation blocks' stored sums), 2 tokens.
    k, n = 256, 16
    w40 = synth.legacy_weights(oracle.TYPE_Q4_0, n, k, 22)
    a = synth.activations(2, k, 23)
    q8 = oracle.q8_1_quantize(a)
    out["q4_0_w"], out["q4_0_x"] = w40, a
    out["q4_0_y"] = oracle.vecq(oracle.TYPE_Q4_0, w40, q8, k, n, tokens=2)
    out["q4_0_sums"] = oracle.vecq_block_sums(oracle.TYPE_Q4_0, w40, q8[:1], k, n)
    # llmp.vecq, IQ4_NL (Q4_0's bytes, ggml's codebook), 2 tokens.
    k, n = 256, 14
    wi = synth.legacy_weights(oracle.TYPE_IQ4_NL, n, k, 26)
    a = synth.activations(2, k, 27)
    q8 = oracle.q8_1_quantize(a)
    out["iq4_nl_w"], out["iq4_nl_x"] = wi, a
    out["iq4_nl_y"] = oracle.vecq(oracle.TYPE_IQ4_NL, wi, q8, k, n, tokens=2)
    out["iq4_nl_sums"] = oracle.vecq_block_sums(oracle.TYPE_IQ4_NL, wi, q8[:1], k, n)
    # llmp.vecq, Q5_K (176-byte super-blocks), 2 tokens.
    k, n = 512, 10
    w5 = synth.q5_k_weights(n, k, 28)
    a = synth.activations(2, k, 29)
    q8 = oracle.q8_1_quantize(a)
    out["q5_k_w"], out["q5_k_x"] = w5, a
    out["q5_k_y"] = oracle.vecq(oracle.TYPE_Q5_K, w5, q8, k, n, tokens=2)
    out["q5_k_sums"] = oracle.vecq_block_sums(oracle.TYPE_Q5_K, w5, q8[:1], k, n)
    # llmp.vecq, Q6_K (210-byte super-blocks), 2 tokens.
    k, n = 512, 12
    w6 = synth.q6_k_weights(n, k, 30)
    a = synth.activations(2, k, 31)
    q8 = oracle.q8_1_quantize(a)
    out["q6_k_w"], out["q6_k_x"] = w6, a
    out["q6_k_y"] = oracle.vecq(oracle.TYPE_Q6_K, w6, q8, k, n, tokens=2)
    out["q6_k_sums"] = oracle.vecq_block_sums(oracle.TYPE_Q6_K, w6, q8[:1], k, n)
    # llmp.vecq, MXFP4 (17-byte blocks), 2 tokens.
    k, n = 512, 12
    wm = synth.mxfp4_weights(n, k, 24)
    a = synth.activations(2, k, 25)
    q8 = oracle.q8_1_quantize(a)
    out["mxfp4_w"], out["mxfp4_x"] = wm, a
    out["mxfp4_y"] = oracle.vecq(oracle.TYPE_MXFP4, wm, q8, k, n, tokens=2)
    out["mxfp4_sums"] = oracle.vecq_block_sums(oracle.TYPE_MXFP4, wm, q8[:1], k, n)
    # llmp.decode.vector: NVFP4 in GGML's blocks with tensor scales, MXFP8 in scale atoms; 3 input rows.
    k, n = 256, 20
    xd = synth.activations(3, k, 26)
    w6 = synth.decode_weight(6, n, k, 27, tensor_scales=2)
    out["dec_x"], out["dec6_data"], out["dec6_tensor_scale"] = xd, w6["data"], w6["tensor_scale"]
    out["dec6_y"] = oracle.decode_vector(6, w6, xd)
    w8a = synth.decode_weight(8, n, k, 28)
    out["dec8_data"], out["dec8_scales"] = w8a["data"], w8a["scales"]
    out["dec8_y"] = oracle.decode_vector(8, w8a, xd, first=3, outputs=11)
    # MXFP8: quantizer and one small product.
    xa = synth.activations(5, 256, 17) * 3.0
    xb = synth.activations(8, 256, 18) * 0.02
    ac, as_ = oracle.mxfp8_quantize(xa)
    bc, bs = oracle.mxfp8_quantize(xb)
    out["mx_a"], out["mx_b"] = xa, xb
    out["mx_a_codes"], out["mx_a_scales"], out["mx_b_codes"], out["mx_b_scales"] = ac, as_, bc, bs
    out["mx_d"] = oracle.mxfp8_gemm(ac, as_, bc, bs)
    # Router.
    logits = synth.activations(4, 16, 19)
    ids, weights = oracle.route(logits, 3)
    out["route_logits"], out["route_ids"], out["route_weights"] = logits, ids, weights
    # EXL3: one 128 x 128 linear at 3 bits, each codebook, 2 rows.
    k = n = 128
    trellis, suh, svh = synth.exl3_weights(k, n, 3, 20)
    xe = synth.activations(2, k, 21).astype(np.float16)
    out["exl3_trellis"], out["exl3_suh"], out["exl3_svh"], out["exl3_x"] = trellis, suh, svh, xe
    for cb in (0, 1, 2):
        out[f"exl3_rotated{cb}"] = oracle.exl3_rotated(trellis, k, n, 3, cb)
        out[f"exl3_y{cb}"] = oracle.exl3_linear(trellis, suh, svh, k, n, 3, cb, xe)
    return out


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vectors.npz")
    np.savez_compressed(path, **build())
    print(path, os.path.getsize(path), "bytes")
