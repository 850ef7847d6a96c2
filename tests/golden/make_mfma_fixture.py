"""Measures what one v_mfma_f32_16x16x128_f8f6f4 returns for chosen E4M3 operands on the GPU of this machine and
writes the measurements as tests/golden/mfma_alignment_gfx950.npz (the committed file was made on an MI355X).

    hipcc -O2 -fPIC -shared --offload-arch=gfx950 -o tests/golden/libmfma_probe.so tests/golden/mfma_probe.hip
    python tests/golden/make_mfma_fixture.py [output.npz]

Families: 1 = two products at chosen k positions (same or different 8-byte runs, all sign combinations), 3 = one large
product and many equal small ones, 4 = random rows (uniform codes, N(0,1)-quantised, sparse).  Every test is one
instruction: A[16][128] and B[16][128] are E4M3 codes by logical k (k = 32 * (lane / 16) + byte of the lane's operand
register), D[i][j] = sum_k A[i][k] * B[j][k] as the instruction returned it with a zero accumulator.
tests/test_oracle_gemm.py checks the oracle's model of the instruction (oracle.gemm_grouped) against the file.
"""
import ctypes, os, sys
import numpy as np, torch
here = os.path.dirname(os.path.abspath(__file__))
lib = ctypes.CDLL(os.path.join(here, "libmfma_probe.so"))
lib.run_probe.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int]
rng = np.random.default_rng(1)
def enc(vals):  # float -> e4m3 code via torch
    return torch.tensor(vals, dtype=torch.float32).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
tests = []  # (family, A[16,128], B[16,128], C[16,16])
Z = lambda: np.zeros((16, 128), np.uint8)
bigs = [0x7e, 0x78, 0x77, 0x70, 0x6b, 0x7e, 0x7d, 0x7c, 0x7b, 0x7a, 0x79, 0x76, 0x75, 0x74, 0x73, 0x72]
smalls_a = [0x7e, 0x70, 0x68, 0x60, 0x58, 0x50, 0x48, 0x44, 0x40, 0x3c, 0x38, 0x34, 0x30, 0x2c, 0x28, 0x20]
smalls_b = [0x38, 0x3a, 0x3c, 0x3e, 0x30, 0x32, 0x28, 0x2b, 0x20, 0x25, 0x18, 0x1f, 0x10, 0x08, 0x04, 0x01]
pairs = [(0, 1), (0, 15), (0, 16), (0, 31), (0, 32), (0, 63), (0, 64), (0, 96), (0, 127), (5, 37), (31, 32), (16, 17), (40, 100), (127, 0), (64, 65), (33, 95)]
# F1: two products, signs
for (p, q) in pairs:
    for sb, ss in ((0, 0), (0, 0x80), (0x80, 0), (0x80, 0x80)):
        A, B = Z(), Z()
        for i in range(16):
            A[i, p] = bigs[i] | sb; A[i, q] = smalls_a[i] | ss
            B[i, p] = bigs[(i * 5) % 16]; B[i, q] = smalls_b[i]
        tests.append((1, A, B, np.zeros((16, 16), np.float32)))
# F3: one big + many equal small ones at set S
sets = {"same32": list(range(1, 32)), "other32": list(range(32, 64)), "all": list(range(1, 128)), "two_groups": list(range(1, 32)) + list(range(64, 96)),
        "eight": list(range(1, 9)), "spread": list(range(4, 128, 4))}
for name, S in sets.items():
    for sign in (0, 0x80):
        A, B = Z(), Z()
        for i in range(16):
            A[i, 0] = bigs[i]; B[i, 0] = bigs[(i * 3) % 16]
            for q in S:
                A[i, q] = smalls_a[i] | sign; B[i, q] = smalls_b[i]
        tests.append((3, A, B, np.zeros((16, 16), np.float32)))
# F4: random rows
finite = np.array([c for c in range(256) if (c & 0x7f) != 0x7f], np.uint8)
for t in range(36):
    kind = t % 6
    if kind < 2:
        A = rng.choice(finite, (16, 128)); B = rng.choice(finite, (16, 128))
    elif kind < 4:
        x = rng.standard_normal((16, 128)); y = rng.standard_normal((16, 128))
        A = enc(x / np.abs(x).max() * 448); B = enc(y / np.abs(y).max() * 448)
    else:  # sparse rows: few non-zeros
        A = np.where(rng.random((16, 128)) < 0.06, rng.choice(finite, (16, 128)), 0).astype(np.uint8)
        B = np.where(rng.random((16, 128)) < 0.5, rng.choice(finite, (16, 128)), 0).astype(np.uint8)
    C = np.zeros((16, 16), np.float32)
    tests.append((4, A.astype(np.uint8), B.astype(np.uint8), C))
fam = np.array([t[0] for t in tests], np.int32)
A = np.stack([t[1] for t in tests]); B = np.stack([t[2] for t in tests]); C = np.stack([t[3] for t in tests])
print("tests", len(tests), flush=True)
dA, dB, dC = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), torch.from_numpy(C).cuda()
dD = torch.zeros_like(dC)
rc = lib.run_probe(dA.data_ptr(), dB.data_ptr(), dC.data_ptr(), dD.data_ptr(), len(tests))
print("rc", rc, flush=True)
out = sys.argv[1] if len(sys.argv) > 1 else os.path.join(here, "mfma_alignment_gfx950.npz")
np.savez_compressed(out, family=fam, A=A, B=B, D=dD.cpu().numpy())
print("wrote", out)
