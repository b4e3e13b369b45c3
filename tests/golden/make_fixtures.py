"""Writes the committed fixtures in this directory.

nibble_kat.json   hand-derived known answers for the AWQ nibble order (worked out on paper
                  from "nibble i stores logical column P[i], P = [0,2,4,6,1,3,5,7]"; they do
                  not come from running any implementation).
awq_small.npz     one seeded small AWQ linear (M=4, K=256, N=64, G=128): inputs, the bits of
                  the dequantised weights and the float64 product, from the pinned CPU oracle.
awq_moe_small.npz one seeded tiny MoE block with its expected output.

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import awq_ref  # noqa: E402


def main():
    kat = {
        "pack": [
            {"logical": [0, 1, 2, 3, 4, 5, 6, 7], "word": "0x75316420", "int32": 0x75316420},
            {"logical": [15, 0, 1, 14, 7, 8, 3, 12], "word": "0xC8E0371F", "int32": -924829921},
            {"logical": [0, 0, 0, 0, 0, 0, 0, 15], "word": "0xF0000000", "int32": -268435456},
        ],
        "unpack": [
            {"word": "0x76543210", "logical": [0, 4, 1, 5, 2, 6, 3, 7]},
            {"word": "0xF0000000", "logical": [0, 0, 0, 0, 0, 0, 0, 15]},
            {"word": "0x0000000F", "logical": [15, 0, 0, 0, 0, 0, 0, 0]},
            {"word": "0x000F0000", "logical": [0, 15, 0, 0, 0, 0, 0, 0]},
        ],
    }
    json.dump(kat, open(os.path.join(HERE, "nibble_kat.json"), "w"), indent=1)

    rng = np.random.default_rng(20240)
    M, K, N, G = 4, 256, 64, 128
    w = rng.integers(0, 16, (K, N))
    z = rng.integers(0, 16, (K // G, N))
    s = (rng.random((K // G, N)) * 0.019 + 0.001).astype(np.float16)
    x = rng.normal(0, 1, (M, K)).astype(np.float16)
    qw, qz = awq_ref.pack_awq(w), awq_ref.pack_awq(z)
    W = awq_ref.dequantize(qw, s, qz, G)
    np.savez_compressed(os.path.join(HERE, "awq_small.npz"), x=x, qweight=qw, scales=s, qzeros=qz,
                        group=np.int64(G), w_dequant_bits=W.view(np.uint16),
                        y_f64=awq_ref.gemm_wide(x, qw, s, qz, G))

    T, H, E, topk, I = 6, 256, 8, 2, 128

    def stack(Kd, Nd):
        ww = rng.integers(0, 16, (E, Kd, Nd))
        zz = rng.integers(0, 16, (E, Kd // G, Nd))
        ss = (rng.random((E, Kd // G, Nd)) * 0.019 + 0.001).astype(np.float16)
        return awq_ref.pack_awq(ww), ss, awq_ref.pack_awq(zz)

    w13, w2 = stack(H, 2 * I), stack(I, H)
    xm = rng.normal(0, 1, (T, H)).astype(np.float16)
    logits = rng.normal(0, 1, (T, E)).astype(np.float32)
    ids, tw = awq_ref.topk_softmax(logits, topk)
    y = awq_ref.moe_forward(xm, w13, w2, ids, tw, G)
    np.savez_compressed(os.path.join(HERE, "awq_moe_small.npz"), x=xm, logits=logits,
                        w13_qweight=w13[0], w13_scales=w13[1], w13_qzeros=w13[2],
                        w2_qweight=w2[0], w2_scales=w2[1], w2_qzeros=w2[2],
                        topk=np.int64(topk), group=np.int64(G), topk_ids=ids, topk_weights=tw, y=y)


if __name__ == "__main__":
    main()
