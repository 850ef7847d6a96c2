"""Grid-search tuner for the FP8 skinny / mid-batch GEMM: measures candidate SgTuning records per
(m, n, k) on the GPU and writes the winners as a tuning table the library loads at run time
(``sg_tuning_load`` / ``rocm_dev_amd.tuning_load``).

This is the run-time counterpart of the reference's grid search: there ``grid.py`` rewrites
``#define`` lines of ``core.cu`` over a fixed search space (grid.py:151-159), drops the points that
do not fit shared memory (skinny_gemm/constraints.py:6-36, 64 KB), recompiles and times each
(grid.py:84-145), and the winner is pasted into the launcher's macro chain
(skinny_gemm/skinny_gemm_caller.cu:86-334).  Here nothing is recompiled: every candidate is one call
of ``sg_skinny_gemm_tuned``; the fit rule is the ring size against gfx950's 160 KB of LDS per CU; and
the result is a text file, one record per shape.

    python -m rocm_dev_amd.autotune --shapes 8x28672x4096 16x4096x14336 --out tuning.txt
    python -m rocm_dev_amd.autotune --preset decode --out tuning.txt --top 3

Only ``search_space`` and the file helpers run without a GPU.
"""
import argparse
import itertools
import sys

LDS_BYTES = 160 * 1024          # per CU on gfx950 (the reference's rule uses 64 KB: constraints.py:11)
LDS_USABLE = LDS_BYTES - 1024   # the kernels keep up to 1 KB of static LDS (arrival word, padding)
VMCNT_MAX = 63                  # outstanding vector-memory instructions a wave can count

ENGINE_DIRECT, ENGINE_LDS, ENGINE_MID = 1, 2, 4
FIELDS = ("engine", "split_k", "waves", "row_tiles", "m_blocks", "depth", "k_chunks", "non_temporal",
          "persistent_wgs_per_cu", "wave_tiles")

PRESETS = {
    # Llama-3-8B projections, decode batch sizes
    "decode": [(m, n, k) for m in (1, 2, 4, 8, 16, 32)
               for (n, k) in ((6144, 4096), (4096, 4096), (28672, 4096), (4096, 14336))],
    # Llama-3-70B-sized layers, mid batch
    "mid": [(m, n, k) for m in (64, 128, 256)
            for (n, k) in ((10240, 8192), (8192, 8192), (57344, 8192), (8192, 28672))],
}
# every dense benchmark shape: what the shipped table (rocm_dev_amd/tuning/mi355x.tbl) is tuned on
PRESETS["baseline"] = PRESETS["decode"] + PRESETS["mid"]


def record(engine, split_k=1, waves=1, row_tiles=1, m_blocks=1, depth=2, k_chunks=4, non_temporal=1,
           persistent_wgs_per_cu=0, wave_tiles=0):
    return dict(zip(FIELDS, (engine, split_k, waves, row_tiles, m_blocks, depth, k_chunks, non_temporal,
                             persistent_wgs_per_cu, wave_tiles)))


def _activation_instructions(m, m_blocks):
    """1 KB activation DMA instructions per 256-byte K stage of the LDS ring (4 rows each)."""
    if m_blocks == 2:
        return 8
    need = (m + 3) // 4
    return 1 if need <= 1 else (2 if need <= 2 else 4)


def lds_ring_fits(m, k, r):
    """The LDS-ring kernels' resource rules for one record: ring + resident activations + reduction
    scratch within LDS, and no more DMA instructions in flight than a wave can count."""
    xu = _activation_instructions(m, r["m_blocks"])
    if k % 256 and not (k % 16 == 0 and k > 256 and ((not r["persistent_wgs_per_cu"] and not r["wave_tiles"] & 7) or r["wave_tiles"] == 1)):
        return False              # part of a block at the end of K: one workgroup per tile, or whole tiles per wave
    blocks = -(-k // 256)
    if r["wave_tiles"] & 8:     # 24-row tiles: two fragments, six weight instructions per stage, one workgroup per tile
        if r["wave_tiles"] != 8 or r["row_tiles"] != 2 or r["persistent_wgs_per_cu"]:
            return False
        return ((r["depth"] - 1) * (6 + xu) <= VMCNT_MAX and r["waves"] * r["depth"] * (6 + xu) * 1024 + 4096 <= LDS_USABLE
                and r["waves"] <= 16 and r["split_k"] <= max(1, blocks))
    frags = r["row_tiles"] * r["m_blocks"]
    mode = r["wave_tiles"] & 3
    resident = mode in (1, 2)
    in_registers = mode == 3
    per_stage = r["row_tiles"] * 4 + (0 if (resident or in_registers) else xu)
    if (r["depth"] - 1) * per_stage > VMCNT_MAX:
        return False
    lds = r["waves"] * r["depth"] * per_stage * 1024 + 4096
    if resident:
        lds += blocks * xu * 1024
    if r["persistent_wgs_per_cu"] and mode != 1:
        lds += 2 * r["waves"] * frags * 1024
    if lds > LDS_USABLE:
        return False
    if in_registers:
        if blocks % r["waves"] or (blocks // r["waves"]) * r["m_blocks"] > 4:
            return False
    if r["wave_tiles"] and (not r["persistent_wgs_per_cu"] or r["split_k"] != 1 or m > 16 * r["m_blocks"]):
        return False
    if r["persistent_wgs_per_cu"] and r["split_k"] != 1:
        return False
    waves = r["waves"] + (1 if r["wave_tiles"] & 4 else 0)
    if waves > 16 or (r["wave_tiles"] & 4 and mode == 1):
        return False
    return r["split_k"] <= max(1, blocks)


def pc_ring_fits(m, k, a_producers, b_producers, consumers, b_lanes, qsize, split_k=1):
    """The producer/consumer ring's resource rules (``sg_skinny_gemm`` with producers > 0): `qsize` slots of
    b_lanes weight tiles + the activation rows of one 256-byte K block, the consumers' double-buffered
    reduction scratch, the flag words and 4 KB of slack within LDS; 1..6 weight tiles per block; no more
    K splits than K blocks."""
    if k % 256 or not 1 <= b_lanes <= 6 or min(a_producers, b_producers, consumers, qsize) < 1:
        return False
    m_blocks = 1 if m <= 16 else 2
    xu = _activation_instructions(m, m_blocks)
    slot = (b_lanes * 4 + xu) * 1024
    flags = -(-((2 * b_lanes * qsize + 2) * 4) // 1024) * 1024
    lds = qsize * slot + 2 * b_lanes * m_blocks * consumers * 1024 + flags + 4096
    return lds <= LDS_USABLE and 1 <= split_k <= k // 256


def mid_fits(k, r):
    """Mid-batch kernel: `depth` weight slots of 16*row_tiles*(waves/2) rows and `k_chunks` (or depth)
    activation slots of 32*m_blocks rows, 128 bytes of K each."""
    wn = r["waves"] // 2
    dx = r["k_chunks"] if 2 <= r["k_chunks"] < r["depth"] else r["depth"]
    bn, bm = 16 * r["row_tiles"] * wn, 32 * r["m_blocks"]
    # (a split whose sum is a second launch, wave_tiles = 1, needs no arrival word)
    if (r["depth"] * bn + dx * bm) * 128 + (16 if r["split_k"] > 1 and r["wave_tiles"] != 1 else 0) > LDS_BYTES:
        return False
    blocks = k // 128
    return r["split_k"] == 1 or blocks // r["split_k"] >= 8


def search_space(m, n, k):
    """Candidate records for one shape, already filtered by the fit rules above.  The library stays the
    authority: a candidate it has no kernel for comes back SG_INVALID_CONFIG and is skipped."""
    out = []
    if m > 32 and (k % 128 == 0 or (k % 16 == 0 and k > 128)):     # (a partial last block: the library has builds for some)
        for waves, rt, mb, depth, dx, sk in itertools.product((4, 8, 14), (2, 4), (2, 4, 8), (2, 3, 4, 6), (0, 2, 3), (1, 2, 3, 4, 5, 6, 8)):
            if dx and dx >= depth:
                continue
            if waves == 14 and rt != 2:             # 224-row tiles: seven waves along n, two fragments each
                continue
            if 32 * mb >= 2 * m and mb > 2:      # tile more than twice as tall as the problem
                continue
            for wt in ((0,) if sk == 1 else (0, 1)):   # a split's sum by the last workgroup to arrive, or by a second launch
                r = record(ENGINE_MID, sk, waves, rt, mb, depth, dx if dx else depth, 1, 0, wt)
                if mid_fits(k, r):
                    out.append(r)
        # the skinny LDS ring over several 32-row activation tiles (what the library runs on small weight matrices)
        if m <= 256 and (k % 256 == 0 or (k % 16 == 0 and k > 256)):
            for sk, waves, rt, depth in itertools.product((1, 2), (1, 2, 3, 4), (1, 2, 4), (2, 3, 4)):
                r = record(ENGINE_LDS, sk, waves, rt, 2, depth, 4, 1, 0, 0)
                if lds_ring_fits(m, k, r):
                    out.append(r)
        return out
    mb = 1 if m <= 16 else 2
    if k % 256 == 0 or (k % 16 == 0 and k > 256):
        for sk, waves, rt, depth, persist, wt in itertools.product((1, 2, 4), (1, 2, 3, 4, 5, 6, 7, 8), (1, 2, 4), (2, 3, 4, 6, 8),
                                                                  (0, 1), (0, 1, 2, 6, 3, 7)):
            if wt and not persist:
                continue
            r = record(ENGINE_LDS, sk, waves, rt, mb, depth, 4, 1, persist, wt)
            if lds_ring_fits(m, k, r):
                out.append(r)
        for sk, waves, depth in itertools.product((1, 2), (1, 2, 4), (2, 3, 4, 6, 8) if mb == 1 else (2, 3, 4)):   # 24-row tiles
            r = record(ENGINE_LDS, sk, waves, 2, mb, depth, 4, 1, 0, 8)
            if lds_ring_fits(m, k, r):
                out.append(r)
    for ku in (1, 2, 4, 8):
        if ku > 1 and k % (64 * ku):
            continue                              # (64-byte stages take any k: the last one may be partial)
        if k % 256 == 0 and ku != 4:
            continue                              # the LDS ring covers these; keep one direct family for comparison
        for sk, waves, rt, depth in itertools.product((1, 2, 4), (1, 2, 4, 8), (1, 2, 3, 4), (1, 2, 4)):
            stages = -(-k // (64 * ku))
            if sk * waves > stages:
                continue
            out.append(record(ENGINE_DIRECT, sk, waves, rt, mb, depth, ku))
    return out


def same_launch(a, b):
    """True if two records describe the same launch: the mid-batch engine reads k_chunks = 0 as "as many
    activation slots as weight slots"."""
    def norm(r):
        r = dict(r)
        if r["engine"] == ENGINE_MID and not 2 <= r["k_chunks"] < r["depth"]:
            r["k_chunks"] = r["depth"]
        return tuple(r[f] for f in FIELDS)
    return norm(a) == norm(b)


def format_table(entries):
    """entries: iterable of ((m, n, k), record dict) -> text of a tuning file."""
    lines = ["sgemm-tuning 1", "# m n k " + " ".join(FIELDS)]
    for (m, n, k), r in sorted(entries):
        lines.append(" ".join(str(v) for v in (m, n, k) + tuple(r[f] for f in FIELDS)))
    return "\n".join(lines) + "\n"


def parse_table(text):
    """Inverse of format_table; raises ValueError on anything sg_tuning_load would reject."""
    entries, header = {}, False
    for raw in text.splitlines():
        line = raw.split("#", 1)[0].strip()
        if not line:
            continue
        if not header:
            if line.split() != ["sgemm-tuning", "1"]:
                raise ValueError("not a version-1 tuning file: %r" % raw)
            header = True
            continue
        v = [int(x) for x in line.split()]
        if len(v) != 3 + len(FIELDS) or min(v[:3]) <= 0 or v[3] not in (ENGINE_DIRECT, ENGINE_LDS, ENGINE_MID):
            raise ValueError("malformed record: %r" % raw)
        entries[tuple(v[:3])] = dict(zip(FIELDS, v[3:]))
    if not header:
        raise ValueError("empty tuning file")
    return entries


# ---- measurement (GPU) ---------------------------------------------------------------------------

class Bench:
    """Operands of one shape on the GPU: enough distinct weight buffers that a launch never finds its
    weights in the 256 MB last-level cache, and the output of the library's own choice to check every
    candidate against."""

    def __init__(self, m, n, k, seed=0):
        import torch
        self.torch = torch
        self.m, self.n, self.k = m, n, k
        g = torch.Generator(device="cuda").manual_seed(seed)
        rot = min(96, max(2, int(640e6 // (n * k)) + 1))
        # N(0, 1) values quantised per tensor to E4M3, the operand distribution of the benchmark configurations: the
        # large mid-batch launches are power-limited, and uniformly random codes (larger magnitudes on average) rank
        # their records differently from real data (256 x 57344 x 8192: an eight-wave record 3 % ahead on uniform
        # codes is 6 % behind on these)
        from . import synth

        def codes(rows):
            return synth.quantize_tensor(torch.randn((rows, k), device="cuda", dtype=torch.float32, generator=g))[0]
        self.weights = [codes(n) for _ in range(rot)]
        self.A = codes(m)
        self.D = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
        self.scale = torch.full((1,), 2.0 ** -10, device="cuda")

    def launch(self, lib, tuning, weight, stream):
        import ctypes as C
        return lib.sg_skinny_gemm_tuned(self.A.data_ptr(), weight.data_ptr(), self.D.data_ptr(), self.scale.data_ptr(),
                                        self.m, self.n, self.k, self.k, C.byref(tuning), stream)

    def time(self, lib, tuning, launches=20, repeats=3):
        """Microseconds per launch, best of `repeats` replays of a graph of `launches` back-to-back launches
        over the weight rotation (at least one launch per buffer: a replay must not find the previous replay's
        weights in the last-level cache); None if the library rejects the record."""
        torch = self.torch
        launches = max(launches, len(self.weights))
        if self.launch(lib, tuning, self.weights[0], torch.cuda.current_stream().cuda_stream) != 0:
            return None
        torch.cuda.synchronize()
        graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                st = torch.cuda.current_stream().cuda_stream
                for i in range(launches):
                    self.launch(lib, tuning, self.weights[i % len(self.weights)], st)
        graph.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        best = float("inf")
        for _ in range(repeats):
            e0.record()
            graph.replay()
            e1.record()
            torch.cuda.synchronize()
            best = min(best, e0.elapsed_time(e1) * 1000.0 / launches)
        return best

    def result(self, lib, tuning):
        torch = self.torch
        rc = self.launch(lib, tuning, self.weights[0], torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        return None if rc != 0 else self.D.float().clone()


def agrees(d, ref, tol=1e-2):
    """The GEMM tolerance of the parity tests: max |d - ref| / max(|ref|, 1e-2 rms(ref)) <= tol."""
    floor = 1e-2 * float(ref.pow(2).mean().sqrt())
    return bool(((d - ref).abs() / ref.abs().clamp_min(floor)).max() <= tol)


def tune_shape(m, n, k, top=1, launches=20, verbose=False, limit=None, finalists=8, rounds=3):
    """Times every candidate of the shape once, then the `finalists` fastest and the library's own choice again in
    `rounds` alternating rounds (one timing after another is repeatable to a few per cent only: the first graphs of
    a process run slow and clocks drift; alternating rounds repeat to a few parts per thousand).  Returns
    ([(us, record)] fastest first by the median over the rounds, candidates whose result disagrees with the
    library's default choice excluded; the default's median; candidates that ran)."""
    import statistics

    from ._lib import lib
    from .api import SgTuning
    bench = Bench(m, n, k)
    default = SgTuning(0, 1, 1, 1, 1, 2, 4, 1, 0, 0)
    ref = bench.result(lib, default)
    if ref is None:
        raise RuntimeError("the library rejects shape %dx%dx%d" % (m, n, k))
    bench.time(lib, default, launches)          # warm-up: the first timed graph of a process is not representative
    timed = []
    space = search_space(m, n, k)
    if limit:
        space = space[:limit]
    for r in space:
        us = bench.time(lib, SgTuning(*(r[f] for f in FIELDS)), launches, repeats=2)
        if us is None:
            continue
        timed.append((us, r))
    timed.sort(key=lambda e: e[0])
    kept = []
    for us, r in timed:                      # verify only as many as go into the final rounds
        d = bench.result(lib, SgTuning(*(r[f] for f in FIELDS)))
        if d is not None and agrees(d, ref):
            kept.append(r)
        elif verbose:
            print("  dropped (result differs): %s" % (r,), file=sys.stderr)
        if len(kept) >= max(top, finalists):
            break
    base, samples = [], [[] for _ in kept]
    for _ in range(max(1, rounds)):
        base.append(bench.time(lib, default, launches))
        for i, r in enumerate(kept):
            samples[i].append(bench.time(lib, SgTuning(*(r[f] for f in FIELDS)), launches))
    final = sorted(((statistics.median(v), r) for v, r in zip(samples, kept)), key=lambda e: e[0])
    return final[:top], statistics.median(base), len(timed)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--shapes", nargs="*", default=[], help="MxNxK ...")
    ap.add_argument("--preset", choices=sorted(PRESETS), action="append", default=[])
    ap.add_argument("--out", required=True, help="tuning file to write")
    ap.add_argument("--merge", help="existing tuning file whose other shapes are kept")
    ap.add_argument("--top", type=int, default=1, help="print this many best candidates per shape")
    ap.add_argument("--launches", type=int, default=20, help="launches per timed graph")
    ap.add_argument("--min-gain", type=float, default=0.02,
                    help="keep a shape out of the table unless the winner beats the built-in choice by this fraction "
                         "(negative: always record the winner, even the built-in choice itself)")
    ap.add_argument("--limit", type=int, default=None, help="time only the first N candidates (smoke runs)")
    ap.add_argument("--report", help="also write what was measured, one JSON object per shape: the built-in choice's and the "
                                     "winner's microseconds, the winner's record, and whether it went into the table")
    args = ap.parse_args(argv)
    shapes = [tuple(int(x) for x in s.lower().split("x")) for s in args.shapes]
    for p in args.preset:
        shapes += PRESETS[p]
    if not shapes:
        ap.error("no shapes: give --shapes and/or --preset")
    entries = parse_table(open(args.merge).read()) if args.merge else {}
    report = []
    for (m, n, k) in shapes:
        kept, base_us, tried = tune_shape(m, n, k, top=max(1, args.top), launches=args.launches, limit=args.limit)
        print("%dx%dx%d: built-in choice %.2f us; %d candidates ran" % (m, n, k, base_us, tried), flush=True)
        for us, r in kept[:args.top]:
            print("   %.2f us  %s" % (us, " ".join("%s=%d" % (f, r[f]) for f in FIELDS)), flush=True)
        # a winner that is the library's own choice under another spelling is timing noise, not a finding
        from .api import skinny_gemm_choice
        own, _ = skinny_gemm_choice(m, n, k)
        own = {f: getattr(own, f) for f in FIELDS}
        if kept and kept[0][0] < base_us * (1.0 - args.min_gain) and (args.min_gain < 0 or not same_launch(kept[0][1], own)):
            entries[(m, n, k)] = kept[0][1]
        else:
            entries.pop((m, n, k), None)
        report.append({"m": m, "n": n, "k": k, "builtin_us": round(base_us, 3), "candidates": tried,
                       "best_us": round(kept[0][0], 3) if kept else None, "best": kept[0][1] if kept else None,
                       "best_is_builtin": bool(kept) and same_launch(kept[0][1], own), "in_table": (m, n, k) in entries})
    with open(args.out, "w") as f:
        f.write(format_table(entries.items()))
    if args.report:
        import json
        with open(args.report, "w") as f:
            f.write("[\n" + ",\n".join(json.dumps(r, sort_keys=True) for r in report) + "\n]\n")
    print("wrote %d record(s) to %s" % (len(entries), args.out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
