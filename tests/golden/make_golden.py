"""Writes the committed golden fixtures (small inputs and the oracle's outputs for them).

Run from the repository root:  python tests/golden/make_golden.py
The fixtures let the GPU tests (and any other implementation) be checked against fixed
vectors without rebuilding inputs: E4M3 decode table, encode probes with ties and
saturation, a dense GEMM case, a 2:4 compress case and a per-row codec case.  Everything
is produced by the CPU oracle, whose functions are pinned by tests/test_oracle_*.py.
"""
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))


def main():
    g = {}
    codes = np.arange(256, dtype=np.uint8)
    g["e4m3_decode_bits"] = [int(b) for b in oracle.e4m3_decode(codes).view(np.uint32)]
    probes = np.array([0.0, -0.0, 1.0, 1.0625, 1.125, 17.0, 19.0, 447.0, 448.0, 463.9, 464.0, 1e9, -1e9, 2.0 ** -10,
                       1.5 * 2.0 ** -9, 2.0 ** -9, 2.0 ** -6, 0.3, -0.7, 3.14159, 250.0, -449.0], dtype=np.float32)
    g["encode_probe_bits"] = [int(b) for b in probes.view(np.uint32)]
    g["encode_probe_codes"] = [int(c) for c in oracle.e4m3_encode(probes)]
    json.dump(g, open(os.path.join(OUT, "formats.json"), "w"), indent=0)

    # dense GEMM: 8 x 64 x 512 from the seeded generator (stream ids as in make_gemm_operands)
    a8, b8, scale = oracle.make_gemm_operands(8, 64, 512, seed=0)
    np.savez_compressed(os.path.join(OUT, "gemm_8x64x512.npz"), a8=a8, b8=b8, scale=np.float32(scale),
                        d_bf16=oracle.gemm_ref(a8, b8, scale), d_f32=oracle.gemm_f32(a8, b8, scale))
    # 2:4: prune + quantise + compress, and the product
    a8, vals, meta, b8, scale = oracle.make_sparse24_operands(8, 32, 512, seed=0)
    np.savez_compressed(os.path.join(OUT, "sparse24_8x32x512.npz"), a8=a8, vals=vals, meta=meta, b8=b8,
                        scale=np.float32(scale), d_bf16=oracle.gemm_sparse24(a8, vals, meta, scale))
    # per-row codec: 16 x 256 with outliers, two buffers, reduce
    xs = [oracle.normal_bf16_outliers((16, 256), seed=i, stream_id=3, frac=0.01, mag=50.0) for i in range(2)]
    enc = [oracle.fp8_encode_rows(x) for x in xs]
    q = np.stack([e[0] for e in enc])
    s = np.stack([e[1] for e in enc])
    np.savez_compressed(os.path.join(OUT, "codec_2x16x256.npz"), x=np.stack(xs), q=q, scales=s,
                        decoded0=oracle.fp8_decode_rows(q[0], s[0]), reduced=oracle.fp8_reduce_rows(q, s))
    print("wrote fixtures to", OUT)


if __name__ == "__main__":
    main()
