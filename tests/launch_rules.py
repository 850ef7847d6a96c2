"""Which explicit configurations the library must run and which it must refuse - written down
independently of the launchers, from the kernels' resource budgets, so that a test can tell a
launcher that wrongly refuses (or wrongly accepts) a configuration from a configuration that
simply does not apply to a shape.  Every function returns the return code the C ABI is expected
to give: 0 (launched), 4 (more than 1024 threads per workgroup) or 6 (no kernel / does not fit).

Budgets on gfx950: 160 KB of LDS per CU, of which the kernels keep 1 KB for static data; a wave
counts at most 63 outstanding vector-memory instructions (vmcnt); a workgroup has at most 1024
threads, and 512 where a wave needs more than 128 registers.
"""
LDS_USABLE = 159 * 1024
VMCNT_MAX = 63
OK, TOO_MANY_WARPS, INVALID = 0, 4, 6


def activation_instructions(m, m_blocks):
    """1 KB DMA instructions that fetch the activation rows of one 256-byte K block (4 rows each,
    rounded up to a compiled count; two 16-row blocks always take 8)."""
    if m_blocks == 2:
        return 8
    need = (m + 3) // 4
    return 1 if need <= 1 else (2 if need <= 2 else 4)


def expect_lds(m, n, k, r):
    """LDS-ring engine (SgTuning.engine = 2) for one record (a dict with autotune.FIELDS keys)."""
    waves, rg, mt, depth, sk = r["waves"], r["row_tiles"], r["m_blocks"], r["depth"], r["split_k"]
    persist, wt = r["persistent_wgs_per_cu"], r["wave_tiles"]
    if k % 256:
        # part of a block at the end of K: only the kernel with one workgroup per tile (16-, 32-, 64- or 24-row tiles)
        if not (k % 16 == 0 and k > 256 and ((persist == 0 and wt & 7 == 0) or wt == 1)):
            return 3
    blocks = k // 256
    if not (1 <= waves <= 16 and depth >= 1 and rg >= 1 and mt in (1, 2) and 1 <= sk <= blocks):
        return INVALID
    if wt & 8:                                            # 24-row tiles: two fragments, six weight instructions per stage
        if rg != 2 or persist != 0 or wt != 8:
            return INVALID
        per_stage = 6 + activation_instructions(m, mt)
        if waves * depth * per_stage * 1024 + 4096 > LDS_USABLE:
            return INVALID
        if waves * 64 > 1024:
            return TOO_MANY_WARPS
        return OK if depth in (2, 3, 4, 6, 8) and (depth - 1) * per_stage <= VMCNT_MAX else INVALID
    xu = activation_instructions(m, mt)
    m_tiles = -(-m // (16 * mt))
    frags = rg * mt
    compiled = rg in (1, 2, 4) and depth in (2, 3, 4, 6, 8)
    wide_regs = 512 if frags >= 8 else 1024              # one workgroup per tile
    wide_regs_persistent = 512 if frags >= 4 else 1024   # persistent kernels recompute addresses: more registers
    if wt == 1:                                           # every wave owns whole tiles, activations resident in LDS
        if sk != 1 or m_tiles != 1 or persist < 1:
            return INVALID
        lds = -(-k // 256) * xu * 1024 + waves * depth * rg * 4096 + 4096
        if lds > LDS_USABLE:
            return INVALID
        if waves * 64 > 1024:
            return TOO_MANY_WARPS
        if not compiled or (depth - 1) * rg * 4 > VMCNT_MAX or waves * 64 > wide_regs_persistent:
            return INVALID
        return OK
    if persist > 0 and wt & 3 == 3:                       # activations in the waves' registers
        if sk != 1 or m_tiles != 1 or blocks % waves:
            return INVALID
        pt = blocks // waves
        if pt * mt > 4:
            return INVALID
        threads = (waves + (1 if wt & 4 else 0)) * 64
        if threads > 1024:
            return TOO_MANY_WARPS
        if waves * depth * rg * 4096 + 2 * waves * frags * 1024 > LDS_USABLE:
            return INVALID
        if depth not in (2, 3, 4) or rg not in (1, 2) or pt not in (1, 2, 4) or (mt == 2 and pt == 4):
            return INVALID
        regs = 16 * pt * mt + 4 * rg * mt + 8 * rg + 40 + 16 * pt * rg
        bound = 1024 if regs <= 100 else (576 if regs <= 160 else 512)
        return OK if threads <= bound else INVALID
    if persist > 0:
        if sk != 1:
            return INVALID
        resident = wt & 3 == 2
        if resident and m_tiles != 1:
            return INVALID
        per_stage = rg * 4 + (0 if resident else xu)
        lds = waves * depth * per_stage * 1024 + 4096 + (blocks * xu * 1024 if resident else 0) + 2 * waves * frags * 1024
        if lds > LDS_USABLE:
            return INVALID
        threads = (waves + (1 if wt & 4 else 0)) * 64
        if threads > 1024:
            return TOO_MANY_WARPS
        if not compiled or (depth - 1) * per_stage > VMCNT_MAX or threads > wide_regs_persistent:
            return INVALID
        return OK
    lds = waves * depth * (rg * 4 + xu) * 1024 + 4096
    if lds > LDS_USABLE:
        return INVALID
    if waves * 64 > 1024:
        return TOO_MANY_WARPS
    if not compiled or (depth - 1) * (rg * 4 + xu) > VMCNT_MAX or waves * 64 > wide_regs:
        return INVALID
    return OK


# (row_tiles, m_blocks, depth, activation slots) the mid-batch kernel is built for, by waves along n
_MID_7 = {(2, 8, 3, 2), (2, 8, 2, 2), (2, 4, 4, 2), (2, 4, 4, 3), (2, 4, 3, 3), (2, 4, 3, 2), (2, 2, 4, 2), (2, 2, 4, 4),
          (2, 2, 3, 3)}
_MID_SAME = {(2, 2, 2), (2, 2, 3), (2, 2, 4), (2, 2, 6), (2, 4, 2), (2, 4, 3), (2, 4, 4), (2, 4, 6), (2, 8, 2), (2, 8, 3),
             (2, 8, 4), (4, 2, 2), (4, 2, 3), (4, 2, 4), (4, 2, 6), (4, 4, 2), (4, 4, 3), (4, 4, 4), (4, 8, 2), (4, 8, 3)}
_MID_DX = {(4, 8, 3, 2), (4, 4, 4, 2), (4, 4, 4, 3), (4, 4, 3, 2), (4, 2, 4, 2), (4, 2, 4, 3), (2, 8, 4, 2), (2, 8, 3, 2),
           (2, 8, 6, 2), (2, 4, 6, 2), (2, 4, 6, 3), (2, 4, 4, 2), (2, 2, 6, 2), (2, 2, 6, 3), (2, 2, 4, 2)}


# (row_tiles, m_blocks, depth, waves along n, activation slots) built with a partial last K block
_MID_TAIL = {(2, 2, 4, 2, 4), (2, 4, 4, 2, 4), (2, 2, 4, 4, 4), (2, 4, 4, 4, 4), (2, 8, 3, 4, 3), (2, 2, 4, 4, 2), (4, 2, 4, 4, 4),
             (4, 2, 3, 4, 3), (4, 4, 3, 4, 3), (4, 8, 3, 4, 2), (4, 8, 2, 4, 2), (2, 2, 4, 7, 4), (2, 4, 4, 7, 3), (2, 8, 3, 7, 2)}


def expect_mid(m, n, k, r):
    """Mid-batch engine (SgTuning.engine = 4): a workgroup tile is 16*row_tiles*(waves/2) weight rows by
    32*m_blocks activation rows, `depth` weight slots and `k_chunks` (or depth) activation slots of
    128 bytes of K."""
    waves, rg, mt, depth, sk, dx = r["waves"], r["row_tiles"], r["m_blocks"], r["depth"], r["split_k"], r["k_chunks"]
    wt = r.get("wave_tiles", 0)
    # a split whose sum is a second launch (wave_tiles = 1) needs no arrival word in LDS
    arrival = 16 if sk > 1 and wt != 1 else 0
    if k % 128:
        # a partial last block: only beyond 128, and only in the builds listed below
        if k % 16 or k <= 128:
            return 3
        if rg not in (2, 4) or mt not in (2, 4, 8) or depth < 2 or waves not in (4, 8, 14):
            return INVALID
        if not 1 <= sk <= k // 128:
            return INVALID
        if wt not in (0, 1):
            return INVALID
        d = dx if 2 <= dx < depth else depth
        wn_ = waves // 2
        if (depth * 16 * rg * wn_ + d * 32 * mt) * 128 + arrival > 160 * 1024:
            return INVALID
        return OK if (rg, mt, depth, wn_, d) in _MID_TAIL else 3
    if rg not in (2, 4) or mt not in (2, 4, 8) or depth < 2 or waves not in (4, 8, 14):
        return INVALID
    wn = waves // 2
    bn, bm = 16 * rg * wn, 32 * mt
    if wn != 7 and bm % (16 * wn):
        return INVALID
    if not 1 <= sk <= k // 128:
        return INVALID
    if wt not in (0, 1):
        return INVALID
    dx = dx if 2 <= dx < depth else depth
    if (depth * bn + dx * bm) * 128 + arrival > 160 * 1024:
        return INVALID
    if wn == 7:
        return OK if (rg, mt, depth, dx) in _MID_7 else INVALID
    if dx == depth:
        if (rg, mt, depth) not in _MID_SAME:
            return INVALID
        if wn == 2 and (depth - 2) * (rg + mt) > VMCNT_MAX:
            return INVALID
        return OK
    return OK if wn == 4 and (rg, mt, depth, dx) in _MID_DX else INVALID


def expect_sparse(m, n, k, r):
    """2:4 engine: stages of 512 k (5 KB per 16 weight rows: 4 KB of values + 1 KB of metadata); k in whole 128-k
    pieces from 512 on, the last stage partly used when 512 does not divide k."""
    waves, rg, mt, depth, sk = r["waves"], r["row_tiles"], r["m_blocks"], r["depth"], r["split_k"]
    persist, wt = r["persistent_wgs_per_cu"], r["wave_tiles"]
    if k < 512 or k % 128:
        return 3
    full, blocks = k // 512, -(-k // 512)
    if mt not in (1, 2) or wt not in (0, 1):
        return INVALID
    if not (1 <= waves <= 16 and depth >= 1 and rg >= 1 and 1 <= sk <= full):
        return INVALID
    need = (m + 3) // 4
    xu2 = 16 if mt == 2 else (2 if need <= 1 else (4 if need <= 2 else 8))
    m_tiles = -(-m // (16 * mt))
    if wt == 1:
        if mt != 1 or m_tiles != 1 or sk != 1 or persist < 1 or rg not in (1, 2):
            return INVALID
        if waves * 64 > 1024:
            return TOO_MANY_WARPS
        if blocks * xu2 * 1024 + waves * depth * rg * 5120 + 8192 > LDS_USABLE:
            return INVALID
        return OK if depth in (2, 3, 4, 6) else INVALID
    if waves * depth * (rg * 5 + xu2) * 1024 + 8192 > LDS_USABLE:
        return INVALID
    if rg not in (1, 2, 4) or depth not in (2, 3, 4, 6) or (depth - 1) * (rg * 5 + xu2) > VMCNT_MAX:
        return INVALID
    if waves * 64 > (512 if (mt == 2 or rg == 4) else 1024):
        return INVALID
    return OK
