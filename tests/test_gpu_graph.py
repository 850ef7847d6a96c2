"""HIP-graph capture and replay of every entry point: a graph is recorded once and replayed several times with
eager work and synchronisations in between, and every replay must reproduce the eager results bit for bit
(split-K included: its arrival counters have to be back at zero after every launch, and the workspace must
already exist - sg_init - because nothing may be allocated during capture)."""
import numpy as np
import pytest
import torch

from gpu_util import dev, scale_tensor

pytestmark = pytest.mark.gpu


def test_replays_match_eager(oracle):
    import rocm_dev_amd as sg
    from rocm_dev_amd._lib import lib
    sg.tuning_clear()
    assert lib.sg_init() == 0
    jobs = []          # (name, launch(), outputs)

    def gemm(m, n, k, seed, tuned=None):
        a8, b8, scale = oracle.make_gemm_operands(m, n, k, seed=seed)
        A, B, S = dev(a8), dev(b8), scale_tensor(scale)
        D = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
        if tuned is None:
            return lambda: sg.skinny_gemm_fastpath(A, B, D, S, check=True), [D]
        return lambda: sg.skinny_gemm_tuned(A, B, D, S, check=True, **tuned), [D]

    jobs.append(("skinny", *gemm(8, 4096, 4096, 1)))
    jobs.append(("persistent", *gemm(8, 8192, 1024, 2)))
    jobs.append(("split-K direct", *gemm(8, 256, 4096, 3, dict(engine=1, split_k=4, waves=4, row_tiles=1, depth=2, k_chunks=4))))
    jobs.append(("split-K ring", *gemm(32, 512, 14336, 4, dict(engine=2, split_k=2, waves=2, row_tiles=2, depth=3))))
    jobs.append(("mid", *gemm(128, 1024, 2048, 5)))
    jobs.append(("mid split-K", *gemm(64, 512, 8192, 6, dict(engine=4, split_k=2, waves=8, row_tiles=2, m_blocks=2, depth=4, k_chunks=2))))
    jobs.append(("mid split-K, sum in a second launch", *gemm(64, 512, 8192, 14, dict(engine=4, split_k=2, waves=8, row_tiles=2, m_blocks=2,
                                                                               depth=4, k_chunks=2, wave_tiles=1))))
    jobs.append(("mid, the library's own six-way split and second launch", *gemm(96, 5120, 13824, 15)))
    # the library's own choices with a K split, several activation tiles, whole tiles per wave and a partial last K block
    jobs.append(("several activation tiles, two K splits", *gemm(40, 1024, 16384, 9)))
    jobs.append(("whole tiles per wave", *gemm(8, 20480, 512, 10)))
    jobs.append(("partial last block", *gemm(8, 2048, 1408, 11)))
    jobs.append(("partial last block, whole tiles per wave", *gemm(16, 20480, 400, 12)))
    jobs.append(("partial last block, mid", *gemm(96, 8192, 400, 13)))

    a8, vals, meta, _, scale = oracle.make_sparse24_operands(8, 1024, 2048, seed=7)
    sA, sV, sM, sS = dev(a8), dev(vals), dev(meta), scale_tensor(scale)
    sD = torch.empty((8, 1024), dtype=torch.bfloat16, device="cuda")
    jobs.append(("sparse", lambda: sg.sparse24_gemm(sA, sV, sM, sD, sS, check=True), [sD]))

    X = dev(oracle.normal_bf16_outliers((64, 2048), seed=8, stream_id=3))
    Q = torch.empty((2, 64, 2048), dtype=torch.uint8, device="cuda")
    Sc = torch.empty((2, 64), dtype=torch.float32, device="cuda")
    Y = torch.empty((64, 2048), dtype=torch.bfloat16, device="cuda")
    Yr = torch.empty((64, 2048), dtype=torch.bfloat16, device="cuda")

    def codec():
        sg.fp8_encode_rows(X, Q[0], Sc[0], check=True)
        sg.fp8_encode_rows(X, Q[1], Sc[1], check=True)
        sg.fp8_decode_rows(Q[0], Sc[0], Y, check=True)
        sg.fp8_reduce_rows(Q, Sc, Yr, check=True)
    jobs.append(("codec", codec, [Q, Sc, Y, Yr]))

    TA = torch.randn((3, 8, 64), device="cuda")
    TB = torch.randn((3, 8, 64), device="cuda")
    TD = torch.empty((8, 64), device="cuda")
    jobs.append(("batch sum", lambda: sg.tiled_sum_reduce(TA, TB, TD, check=True), [TD]))

    def snapshot():
        torch.cuda.synchronize()
        return [[o.clone() for o in outs] for _, _, outs in jobs]

    def poison():
        for _, _, outs in jobs:
            for o in outs:
                o.view(torch.uint8).fill_(0xA5)

    for _, launch, _ in jobs:
        launch()
    eager = snapshot()

    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for _, launch, _ in jobs:
                launch()
    for replay in range(4):
        poison()
        (torch.randn((1024, 1024), device="cuda") @ torch.randn((1024, 1024), device="cuda")).sum().item()   # eager work between replays
        graph.replay()
        got = snapshot()
        for (name, _, _), want_outs, got_outs in zip(jobs, eager, got):
            for w, g in zip(want_outs, got_outs):
                assert torch.equal(w.view(torch.uint8), g.view(torch.uint8)), (name, replay)
    # and the eager path still works after the replays (split-K counters were left at zero)
    poison()
    for _, launch, _ in jobs:
        launch()
    for (name, _, _), want_outs, got_outs in zip(jobs, eager, snapshot()):
        for w, g in zip(want_outs, got_outs):
            assert torch.equal(w.view(torch.uint8), g.view(torch.uint8)), (name, "eager after replays")
