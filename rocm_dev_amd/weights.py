"""On-disk container for the FP8 weights the GEMM entry points read: dense OCP-E4M3 matrices and their 2:4
compressed form (values + position nibbles, the layout documented for ``sg_sparse24_gemm`` in include/sgemm.h).

No counterpart in the reference, whose harness regenerates random operands on every run (common.cuh:86-105);
this is the storage side of the 2:4 path: prune + compress once (on the GPU, ``sg_sparse24_compress``), keep the
result, load it straight into device memory.

File layout, little endian, version 1::

    0   4  magic  b"SGW8"
    4   4  version (1)
    8   4  kind    1 = dense [n][k] E4M3 codes, 2 = 2:4 compressed (values [n][k/2], then metadata [n][k/8])
    12  4  n       weight rows (output features)
    16  4  k       dense K (input features)
    20  4  tensor scale, float32 (the per-tensor factor the codes were quantised with; 1.0 if none)
    24  8  bytes of the first payload (dense codes, or the 2:4 values)
    32  8  bytes of the second payload (2:4 metadata; 0 for dense)
    40  4  CRC-32 of both payloads, in file order
    44 20  zero
    64     first payload, then the second, each starting on a 64-byte boundary

    python -m rocm_dev_amd.weights compress dense.sgw8 sparse.sgw8     # prune 2:4 + compress on the GPU
    python -m rocm_dev_amd.weights info sparse.sgw8
"""
import argparse
import struct
import sys
import zlib

import numpy as np

MAGIC = b"SGW8"
VERSION = 1
KIND_DENSE, KIND_SPARSE24 = 1, 2
HEADER = struct.Struct("<4sIIIIfQQI20x")
assert HEADER.size == 64


def _pad(nbytes):
    return (-nbytes) % 64


class WeightFileError(ValueError):
    """The file is not a weight container this version reads (bad magic, version, sizes or checksum)."""


def _as_u8(a, shape, what):
    a = np.ascontiguousarray(np.asarray(a))
    if a.dtype != np.uint8 or a.shape != shape:
        raise ValueError("%s must be uint8 of shape %s, got %s %s" % (what, shape, a.dtype, a.shape))
    return a


def _write(path, kind, n, k, scale, first, second):
    crc = zlib.crc32(first.tobytes())
    crc = zlib.crc32(second.tobytes(), crc) if second is not None else crc
    with open(path, "wb") as f:
        f.write(HEADER.pack(MAGIC, VERSION, kind, n, k, float(scale), first.nbytes,
                            0 if second is None else second.nbytes, crc & 0xFFFFFFFF))
        f.write(first.tobytes())
        f.write(b"\0" * _pad(first.nbytes))
        if second is not None:
            f.write(second.tobytes())
            f.write(b"\0" * _pad(second.nbytes))


def save_dense(path, codes, scale=1.0):
    """codes: [n][k] uint8 OCP-E4M3 (numpy array or CPU/GPU torch tensor)."""
    codes = _to_numpy(codes)
    if codes.ndim != 2 or codes.shape[1] % 16:
        raise ValueError("dense weights must be [n][k] with k a multiple of 16")
    n, k = codes.shape
    _write(path, KIND_DENSE, n, k, scale, _as_u8(codes, (n, k), "codes"), None)


def save_sparse24(path, vals, meta, scale=1.0):
    """vals [n][k/2], meta [n][k/8] uint8, as sg_sparse24_compress writes them."""
    vals, meta = _to_numpy(vals), _to_numpy(meta)
    if vals.ndim != 2 or meta.ndim != 2 or vals.shape[0] != meta.shape[0] or vals.shape[1] != 4 * meta.shape[1]:
        raise ValueError("2:4 weights must be values [n][k/2] and metadata [n][k/8]")
    n, k = vals.shape[0], 2 * vals.shape[1]
    if k % 16:
        raise ValueError("k must be a multiple of 16")
    _write(path, KIND_SPARSE24, n, k, scale, _as_u8(vals, (n, k // 2), "vals"), _as_u8(meta, (n, k // 8), "meta"))


def _to_numpy(a):
    if hasattr(a, "detach"):                 # torch tensor; float8 is viewed as its codes
        import torch
        if a.dtype == torch.float8_e4m3fn:
            a = a.view(torch.uint8)
        return a.detach().cpu().numpy()
    return np.asarray(a)


def read_header(path):
    """dict(kind, n, k, scale, first_bytes, second_bytes, crc) after checking everything the header alone can tell."""
    with open(path, "rb") as f:
        raw = f.read(HEADER.size)
        f.seek(0, 2)
        size = f.tell()
    if len(raw) < HEADER.size:
        raise WeightFileError("%s: shorter than the 64-byte header" % path)
    magic, version, kind, n, k, scale, first, second, crc = HEADER.unpack(raw)
    if magic != MAGIC:
        raise WeightFileError("%s: not a weight container (magic %r)" % (path, magic))
    if version != VERSION:
        raise WeightFileError("%s: version %d, this reader knows version %d" % (path, version, VERSION))
    if kind not in (KIND_DENSE, KIND_SPARSE24) or n <= 0 or k <= 0 or k % 16:
        raise WeightFileError("%s: bad kind/shape (%d, %d x %d)" % (path, kind, n, k))
    want = (n * k, 0) if kind == KIND_DENSE else (n * (k // 2), n * (k // 8))
    if (first, second) != want:
        raise WeightFileError("%s: payload sizes %d + %d do not match a %d x %d matrix of kind %d" % (path, first, second, n, k, kind))
    need = HEADER.size + first + _pad(first) + (second + _pad(second) if second else 0)
    if size < need:
        raise WeightFileError("%s: truncated (%d bytes, need %d)" % (path, size, need))
    return dict(kind=kind, n=n, k=k, scale=scale, first_bytes=first, second_bytes=second, crc=crc)


def load(path, device=None, verify=True):
    """Reads a container.  Returns dict(kind, n, k, scale, codes) for dense files and dict(kind, n, k, scale, vals,
    meta) for 2:4 files; the matrices are read-only numpy memory maps when ``device`` is None, torch uint8 tensors
    on ``device`` otherwise.  ``verify`` checks the payload checksum (one pass over the file)."""
    h = read_header(path)
    n, k = h["n"], h["k"]
    off0 = HEADER.size
    mode = "r" if device is None else "c"     # torch wants writable memory to copy from; "c" never touches the file
    if h["kind"] == KIND_DENSE:
        parts = {"codes": np.memmap(path, np.uint8, mode, off0, (n, k))}
    else:
        off1 = off0 + h["first_bytes"] + _pad(h["first_bytes"])
        parts = {"vals": np.memmap(path, np.uint8, mode, off0, (n, k // 2)),
                 "meta": np.memmap(path, np.uint8, mode, off1, (n, k // 8))}
    if verify:
        crc = 0
        for a in parts.values():
            crc = zlib.crc32(a, crc)
        if crc & 0xFFFFFFFF != h["crc"]:
            raise WeightFileError("%s: payload checksum mismatch" % path)
    out = dict(kind=h["kind"], n=n, k=k, scale=h["scale"])
    if device is None:
        out.update(parts)
    else:
        import torch
        for name, a in parts.items():
            out[name] = torch.from_numpy(a).to(device)
    return out


def compress_file(dense_path, sparse_path, device="cuda"):
    """Dense container -> 2:4 container: prune (two largest magnitudes of every four codes, ties to the lower
    position) and compress on the GPU with sg_sparse24_compress.  The tensor scale is carried over."""
    import torch

    from . import api
    w = load(dense_path, device=device)
    if w["kind"] != KIND_DENSE:
        raise WeightFileError("%s is not a dense container" % dense_path)
    n, k = w["n"], w["k"]
    vals = torch.empty((n, k // 2), dtype=torch.uint8, device=device)
    meta = torch.empty((n, k // 8), dtype=torch.uint8, device=device)
    api.sparse24_compress(w["codes"], vals, meta, check=True)
    torch.cuda.synchronize()
    save_sparse24(sparse_path, vals, meta, w["scale"])
    return n, k


def main(argv=None):
    ap = argparse.ArgumentParser(description="FP8 weight containers for libsgemm")
    sub = ap.add_subparsers(dest="cmd", required=True)
    c = sub.add_parser("compress", help="dense container -> 2:4 container (needs the GPU)")
    c.add_argument("dense")
    c.add_argument("sparse")
    i = sub.add_parser("info", help="print the header and verify the checksum")
    i.add_argument("path")
    args = ap.parse_args(argv)
    if args.cmd == "compress":
        n, k = compress_file(args.dense, args.sparse)
        print("%s: %d x %d, %.3f bytes per dense weight" % (args.sparse, n, k, 0.625))
    else:
        h = read_header(args.path)
        load(args.path, verify=True)
        print("%s: %s %d x %d, scale %g, payload %d + %d bytes, checksum ok"
              % (args.path, "dense" if h["kind"] == KIND_DENSE else "2:4", h["n"], h["k"], h["scale"], h["first_bytes"], h["second_bytes"]))
    return 0


if __name__ == "__main__":
    sys.exit(main())
