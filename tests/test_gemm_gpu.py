"""
GPU parity tests of the mixed INT4/FP6 GEMM, through the C ABI (fp6_marlin.mul -> libfp6m.so:fp6m_mul).

Oracle: dequantise-then-matmul (test.py:165-167) on operands quantised and packed by the CPU oracle;
tolerance mean|C - C_ref| / mean|C_ref| <= 1e-3 (test.py:181).  The five groups of the reference's test.py
are reproduced (tiles, k divisibility, very few k steps, errors, mixed), then group-128 scales, the
the benchmark's configurations (Llama-2 layer shapes, the M sweep), forced split-k reductions, and bit-exact one-hot probes that pin the layout at
any size.
"""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TOL = 1e-3   # test.py:181
_cache = {}


def dev():
    return torch.device("cuda:0")


def problem(oracle, n, k, qc=-1, gs=-1, seed=0):
    """Packed operands from the *oracle* (cached per shape): (w_ref np f16 [k,n], B cuda int32, s cuda f16)."""
    key = (n, k, qc, gs, seed)
    if key not in _cache:
        rng = np.random.default_rng(seed + 1000 * n + k)
        w = rng.normal(0, 0.02, (k, n)).astype(np.float16)
        ref, b, s = oracle.gen_mixed_weight(w, qc, gs, strict=False)
        _cache[key] = (ref, torch.from_numpy(b).to(dev()), torch.from_numpy(s).to(dev()))
    return _cache[key]


def run(oracle, m, n, k, thread_k=-1, thread_n=-1, qc=-1, gs=-1, seed=0, max_par=16, ksplit=None, sms=-1, env=None):
    import fp6_marlin
    print(f"case m={m} n={n} k={k} tk={thread_k} tn={thread_n} qc={qc} gs={gs} ksplit={ksplit} sms={sms} env={env}", flush=True)
    knobs = {name[5:].lower(): value for name, value in (env or {}).items()}    # FP6M_WK -> wk
    ref, B, s = problem(oracle, n, k, qc, gs, seed)
    g = torch.Generator().manual_seed(seed * 7919 + m)
    A = torch.randn((m, k), generator=g, dtype=torch.float32).half()
    C = torch.full((m, n), float("nan"), dtype=torch.half, device=dev())      # must be fully overwritten
    ws = torch.zeros(n // 128 * max_par, dtype=torch.int32, device=dev())
    if ksplit is not None:
        knobs["ksplit"] = ksplit
    with fp6_marlin.cabi.tuning(**knobs):                           # overrides of the dispatcher's choices
        fp6_marlin.mul(A.to(dev()), B, C, s, ws, qc, thread_k, thread_n, sms, max_par, gs)
        torch.cuda.synchronize()
        C2 = torch.full_like(C, float("nan"))                          # same call again: results are reproducible
        fp6_marlin.mul(A.to(dev()), B, C2, s, ws, qc, thread_k, thread_n, sms, max_par, gs)
        torch.cuda.synchronize()
    assert int(ws.abs().sum().item()) == 0, "workspace must be left zeroed"
    c = C.cpu().numpy()
    assert np.isfinite(c).all(), "C not fully written"
    assert torch.equal(C, C2), "two identical calls differ"
    c_ref = oracle.matmul_ref(A.numpy(), ref)
    err = oracle.rel_err(c, c_ref)
    assert err <= TOL, f"rel err {err}"
    # the same bar on each region alone: an error confined to the few FP6 columns must not hide in the overall mean
    n6 = qc if qc > 0 else 0
    for name, sl in (("INT4", slice(0, n - n6)), ("FP6", slice(n - n6, n))):
        if sl.stop > sl.start:
            e = oracle.rel_err(c[:, sl], c_ref[:, sl])
            assert e <= TOL, f"rel err {e} on the {name} columns"
    return c


# ------------------------------------------------------------------ the reference's five test groups

def test_tiles(oracle):                                            # test.py:183-190
    for m in [1, 2, 3, 4, 8, 12, 16, 24, 32, 48, 64, 118, 128, 152, 768, 1024]:
        for tk, tn in [(64, 256), (128, 128)]:
            if m > 16 and tk == 128:
                continue
            run(oracle, m, 512, 1024, tk, tn)


def test_k_stages_divisibility(oracle):                            # test.py:192-195
    for k in [3 * 64 + 64 * 4 * 2 + 64 * i for i in range(1, 4)]:
        run(oracle, 16, 512, k, 64, 256)


def test_very_few_stages(oracle):                                  # test.py:197-200
    for k in [64, 128, 192]:
        run(oracle, 16, 512, k, 64, 256)


def test_errors(oracle):                                           # test.py:202-227
    import fp6_marlin
    m, n, k = 16, 256, 64
    ref, B, s = problem(oracle, n, k)
    A = torch.randn((m, k), dtype=torch.half, device=dev())
    C = torch.zeros((m, n), dtype=torch.half, device=dev())
    small_ws = torch.zeros(n // 128, dtype=torch.int32, device=dev())
    ws = torch.zeros(n // 128 * 16, dtype=torch.int32, device=dev())
    with pytest.raises(RuntimeError):                              # workspace too small (fp6_marlin_cuda.cpp:62-63)
        fp6_marlin.mul(A, B, C, s, small_ws, -1, 128, 128, -1)
    with pytest.raises(RuntimeError, match="not compatible"):      # k=64 with thread_k=128
        fp6_marlin.mul(A, B, C, s, ws, -1, 128, 128, -1)
    with pytest.raises(RuntimeError, match="No kernel"):           # no 256x256 kernel
        ref2, B2, s2 = problem(oracle, 256, 256)
        A2 = torch.randn((m, 256), dtype=torch.half, device=dev())
        fp6_marlin.mul(A2, B2, C, s2, ws, -1, 256, 256, -1)
    with pytest.raises(RuntimeError):                              # scales of shape (2, n)
        fp6_marlin.mul(A, B, C, torch.zeros((2, n), dtype=torch.half, device=dev()), ws, -1, 64, 256, -1)
    with pytest.raises(RuntimeError):                              # CPU tensor
        fp6_marlin.mul(A.cpu(), B, C, s, ws)
    torch.cuda.synchronize()


def test_mixed(oracle):                                            # test.py:229-237
    for m in [1, 12, 16, 64, 65, 77, 152, 256, 1024]:
        for n, k in [(256, 512), (256 * 2, 1024), (256 * 100, 1024)]:
            for tk, tn in [(128, 128), (64, 256)]:
                if m > 16 and tk == 128:
                    continue
                run(oracle, m, n, k, tk, tn, qc=256)


# ------------------------------------------------------------------ beyond the reference's kernel

def test_group128_scales(oracle):
    for m in [1, 16, 33, 64, 200]:
        run(oracle, m, 512, 1024, qc=-1, gs=128)
        run(oracle, m, 768, 512, qc=256, gs=128)


def test_quant_cols_other_than_256(oracle):
    for qc in [128, 512]:
        for m in [1, 16, 40]:
            run(oracle, m, 1024, 512, qc=qc)
            run(oracle, m, 1024, 512, qc=qc, gs=128)


def test_forced_split_k_and_determinism(oracle):
    """Cross-workgroup reduction with 1, 2, 3, 8 and 16 partners, repeated runs bit-identical."""
    for m in [1, 16, 64]:
        outs = []
        for ks in [1, 2, 3, 8, 16]:
            outs.append(run(oracle, m, 512, 2048, qc=256, ksplit=ks))
        again = run(oracle, m, 512, 2048, qc=256, ksplit=8)
        assert np.array_equal(again.view(np.uint16), outs[3].view(np.uint16))
    run(oracle, 16, 512, 2048, qc=256, sms=1)                       # `sms` caps the partners at one


def test_cells_and_partial_tiles_up_to_sixteen_rows(oracle):
    """The m <= 16 kernel sums a tile shared by several workgroups in the accumulate-and-count cells up to four rows
    and through published partial tiles gathered by the last arrival beyond (the `cells` knob sends the small row
    counts there too): every row count class, 1 .. 16 partners, both scale modes, all FP6, one-hot rows bit for
    bit, each against itself on a second call, and the two paths against each other."""
    for cells in (1, 0):
        e = {"FP6M_CELLS": cells}
        for m in (2, 3, 4, 5, 9, 16):
            run(oracle, m, 512, 2048, qc=256, gs=128, env=e)
            run(oracle, m, 1024, 1024, qc=256, ksplit=3, env=e)
        for ks in (2, 8, 16):
            run(oracle, 4, 512, 2048, qc=256, ksplit=ks, env=e)
            run(oracle, 16, 512, 2048, qc=256, ksplit=ks, env=e)
        run(oracle, 3, 256, 4096, qc=-1, env=e)
        run(oracle, 4, 512, 1024, qc=512, ksplit=4, env=e)                 # all FP6
        for gs in (-1, 128):
            one_hot_case(oracle, 4, 768, 1024, 256, gs, {"cells": cells, "ksplit": 4})
            one_hot_case(oracle, 3, 512, 2048, 256, gs, {"cells": cells})
    # the same sums either way, up to the cells' fixed-point grid of 2^-29 in output units: at most one fp16 ulp apart
    a = run(oracle, 4, 512, 2048, qc=256, gs=128, ksplit=8, env={"FP6M_CELLS": 1})
    b = run(oracle, 4, 512, 2048, qc=256, gs=128, ksplit=8, env={"FP6M_CELLS": 0})
    ulps = np.abs(a.view(np.int16).astype(np.int32) - b.view(np.int16).astype(np.int32))
    assert ulps.max() <= 1 and (ulps != 0).mean() < 0.01, (ulps.max(), (ulps != 0).mean())


def test_partial_tiles_exchanged_through_one_xcd(oracle):
    """5 .. 16 rows: the workgroups that share a tile may be placed on one XCD and exchange their partial tiles through its
    L2 (`xcd` knob: 1 forces the placement, 0 the agent-scope exchange).  Same sums in the same order: the results
    must agree bit for bit -- for tile counts that do and do not divide by the eight XCDs, several split factors
    (forced and the dispatcher's own), both scale modes, all FP6; on the default stream, on a side stream and from a
    replayed HIP graph (the XCD that a dispatch's first workgroup runs on differs between them)."""
    import fp6_marlin
    for (m, n, k, qc, gs, ks) in [(16, 512, 2048, 256, 128, None), (16, 1024, 2048, 256, -1, 4), (5, 1280, 1024, 256, 128, 3),
                                  (9, 2304, 1024, 512, 128, 2), (16, 4096, 1024, 256, 128, None), (8, 512, 2048, 512, -1, 6),
                                  (16, 1152, 4096, 128, 128, 16), (12, 3072, 512, 256, -1, 2)]:
        a = run(oracle, m, n, k, qc=qc, gs=gs, ksplit=ks, env={"FP6M_XCD": 0})
        b = run(oracle, m, n, k, qc=qc, gs=gs, ksplit=ks, env={"FP6M_XCD": 1})
        assert np.array_equal(a.view(np.uint16), b.view(np.uint16)), (m, n, k, qc, gs, ks)
    one_hot_case(oracle, 16, 1024, 2048, 256, 128, {"xcd": 1, "ksplit": 4})
    one_hot_case(oracle, 7, 768, 1024, 256, -1, {"xcd": 1, "ksplit": 2})
    # other streams, and a captured graph replayed several times with eager work in between
    m, n, k, qc, gs = 16, 2048, 2048, 256, 128
    ref, B, s = problem(oracle, n, k, qc, gs)
    A = torch.randn((m, k), generator=torch.Generator().manual_seed(5), dtype=torch.float32).half().to(dev())
    ws = fp6_marlin.init_workspace(torch.zeros(n // 128 * 16, dtype=torch.int32, device=dev()))
    outs = {}
    for xcd in (0, 1):
        with fp6_marlin.cabi.tuning(xcd=xcd, ksplit=4):
            C = torch.full((m, n), float("nan"), dtype=torch.half, device=dev())
            fp6_marlin.mul(A, B, C, s, ws, qc, -1, -1, -1, 16, gs)
            torch.cuda.synchronize()
            outs[xcd] = C.clone()
            side = torch.cuda.Stream()
            with torch.cuda.stream(side):
                C.fill_(float("nan"))
                fp6_marlin.mul(A, B, C, s, ws, qc, -1, -1, -1, 16, gs)
            side.synchronize()
            assert torch.equal(C, outs[xcd]), f"side stream, xcd={xcd}"
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                fp6_marlin.mul(A, B, C, s, ws, qc, -1, -1, -1, 16, gs)
            for _ in range(3):
                C.fill_(float("nan"))
                graph.replay()
                torch.cuda.synchronize()
                assert torch.equal(C, outs[xcd]), f"graph replay, xcd={xcd}"
                C.fill_(float("nan"))
                fp6_marlin.mul(A, B, C, s, ws, qc, -1, -1, -1, 16, gs)   # eager, after a capture
                torch.cuda.synchronize()
                assert torch.equal(C, outs[xcd]), f"eager after capture, xcd={xcd}"
    assert torch.equal(outs[0], outs[1])
    assert int(ws.abs().sum().item()) == 0
    c_ref = oracle.matmul_ref(A.cpu().numpy(), ref)
    assert oracle.rel_err(outs[1].cpu().numpy(), c_ref) <= TOL


def test_two_classes_of_int4_tiles(oracle, capfd):
    """The m <= 16 kernel with the INT4 tiles in two classes (as many whole tiles as fill the CUs once, the rest in
    parts on later workgroups), forced onto small problems by pretending a chip of a few CUs: cells (up to four rows)
    and partial tiles (beyond), both scale modes, with and without an FP6 region, the second class whole or in two
    parts; and one-hot rows bit for bit.  The second identical call inside run() also checks that counters and cells
    are left clean."""
    import re
    cases = [(8, 1536, 2048, 256), (9, 1536, 2048, 256), (12, 2304, 2048, 256), (16, 3072, 1024, -1), (20, 3072, 1024, -1)]
    for cus, n, k, qc in cases:
        e = {"FP6M_CLS": 1, "FP6M_CUS": cus, "FP6M_VERBOSE": 1}
        for m in (2, 4, 5, 16):
            for gs in (-1, 128):
                run(oracle, m, n, k, qc=qc, gs=gs, env=e)
        out = capfd.readouterr().err
        second = [int(x) for x in re.findall(r"\(\+ (\d+) tiles in \d+ parts\)", out)]
        assert len(second) == 16 and all(x > 0 for x in second), out[-3000:]
        for gs in (-1, 128):
            for m in (3, 9, 16):
                one_hot_case(oracle, m, n, k, qc, gs, {"cls": 1, "cus": cus})


def test_two_classes_of_int4_tiles_beyond_sixteen_rows(oracle, capfd):
    """The m > 16 kernel's plan for one row tile and somewhat more tiles than CUs (as many whole tiles as there are CUs,
    the rest in parts on the grid's last workgroups), forced onto small problems by pretending a chip of a few CUs:
    32-row tiles with both scale modes, 64-row tiles with group scales, the second class in one and in two parts, with
    and without an FP6 region; and one-hot rows bit for bit."""
    import re
    cases = [(8, 1536, 2048, 256, 128), (8, 1536, 4096, 256, 128), (16, 3072, 4096, -1, 128), (8, 1536, 2048, 256, -1),
             (16, 3072, 2048, -1, -1)]
    for cus, n, k, qc, gs in cases:
        e = {"FP6M_CLS": 1, "FP6M_CUS": cus, "FP6M_VERBOSE": 1}
        rows = (17, 32, 40, 64) if gs == 128 else (17, 32)
        for m in rows:
            run(oracle, m, n, k, qc=qc, gs=gs, env=e)
        out = capfd.readouterr().err
        second = [int(x) for x in re.findall(r"MB=\d row tiles 1 .*\(\+ (\d+) tiles in \d+ parts\)", out)]
        assert len(second) == 2 * len(rows) and all(x > 0 for x in second), out[-3000:]
        for m in rows[1::2]:
            one_hot_case(oracle, m, n, k, qc, gs, {"cls": 1, "cus": cus})


def test_eight_row_blocks_per_wave(oracle):
    """The m > 16 kernel with eight 16-row blocks per wave (128-row tiles, accumulators in the accumulation
    registers), forced onto small problems: ragged row tiles, both regions, both scale modes, k splits through the
    scratch, several launches, and one-hot rows bit for bit."""
    for pair in (1,):                                                   # (eight blocks always fetch A by pairs of steps)
        e = {"FP6M_MB": 8, "FP6M_PAIR": pair}
        for m in (17, 100, 128, 129, 300):
            run(oracle, m, 512, 1024, qc=256, gs=128, env=e)
            run(oracle, m, 512, 1024, qc=256, env=e)
        run(oracle, 200, 768, 512, qc=128, env=e)
        run(oracle, 130, 256, 64, qc=-1, env=e)                         # one k unit: three idle slices
        run(oracle, 260, 512, 2048, qc=256, gs=128, ksplit=3, env=e)
        run(oracle, 520, 512, 512, qc=512, ksplit=2, env=e)             # all FP6
        run(oracle, 2100, 256, 1024, qc=-1, gs=128, max_par=16, env=e)  # second launch of 52 rows
        for n, k, qc in [(512, 256, 256), (768, 1024, 256)]:
            for gs in (-1, 128):
                one_hot_case(oracle, 200, n, k, qc, gs, {"mb": 8, "pair": pair})
                one_hot_case(oracle, 130, n, k, qc, gs, {"mb": 8, "ksplit": 2, "pair": pair})


def test_dispatch_picks_128_row_tiles_where_they_fill_the_chip(oracle, capfd):
    """The dispatcher's own choice between 128-row tiles (one workgroup per CU, whole rounds) and 64-row tiles (a third
    slower per row, finer grain): with 32 column tiles, 8 row tiles of 128 fill one round of 256 CUs exactly (the last
    tile ragged at m = 1000) and 5 of them beat 10 half-size workgroups that no longer fit one per CU; 9 row tiles
    would take two rounds for 1.1 rounds of work, and at m = 300 the 64-row tiles still fit one per CU.  With 256
    column tiles even a single, ragged row tile of 128 wins (one round instead of 512 half-size workgroups)."""
    for m, n, want in ((1000, 4096, "MB=8"), (1024, 4096, "MB=8"), (640, 4096, "MB=8"), (1025, 4096, "MB=4"),
                       (300, 4096, "MB=4"), (96, 32768, "MB=8"), (96, 4096, "MB=4"), (64, 32768, "MB=4")):
        capfd.readouterr()
        run(oracle, m, n, 512, qc=256, gs=128, env={"FP6M_VERBOSE": 1})
        err = capfd.readouterr().err
        assert want in err, (m, n, want, err[-400:])


def test_eight_k_slices_per_workgroup(oracle):
    """The m > 16 kernel with eight waves (k slices) per workgroup, which small grids on long k pick by themselves
    (here: 8192 x 512 at m = 40), forced on and off on ragged shapes."""
    for wk in (8, 4):
        e = {"FP6M_WK": wk}
        for m in (17, 32, 33, 64, 100, 200):
            run(oracle, m, 512, 1024, qc=256, gs=128, env=e)
        run(oracle, 48, 768, 512, qc=128, env=e)
        run(oracle, 70, 256, 64, qc=-1, env=e)                          # one k unit: seven idle slices
        run(oracle, 130, 512, 2048, qc=256, ksplit=3, env=e)
    run(oracle, 40, 512, 8192, qc=256, gs=128)


def test_paired_activation_fetch_of_the_four_block_kernel(oracle):
    """The m > 16 kernel with the activations fetched a pair of k steps at a time and the packed words through
    registers (picked from 33 rows on, and for 32-row tiles in eight-wave workgroups), forced on and off: ragged row counts (row groups of eight that are partly
    or wholly past m), one k unit per slice, group scales or not, FP6-only and INT4-only problems, eight or four
    slices per workgroup, several launches."""
    for pair in (1, 0):
        for wk in (8, 4):
            e = {"FP6M_PAIR": pair, "FP6M_WK": wk}
            for m in (33, 41, 64, 65, 100, 128, 199):
                run(oracle, m, 512, 1024, qc=256, gs=128, env=e)
            run(oracle, 48, 768, 512, qc=128, env=e)
            run(oracle, 70, 256, 64, qc=-1, env=e)                      # one k unit: idle slices
            run(oracle, 130, 512, 2048, qc=256, ksplit=3, env=e)
            run(oracle, 77, 512, 512, qc=512, ksplit=2, env=e)          # all FP6
            run(oracle, 300, 256, 1024, qc=-1, gs=128, max_par=2, env=e)   # three launches, the last of 44 rows
    run(oracle, 256, 2048, 2048, qc=256, gs=128)                        # the dispatcher's own choice of it
    # 32-row tiles take the paired loop in eight-wave workgroups (two blocks per step walk the four activation
    # register buffers in two steps): ragged rows, both scale modes, all FP6, a forced split, one-hot rows bit for
    # bit, and bit-identical to the ring loop
    for m in (17, 24, 25, 32):
        outs = [run(oracle, m, 512, 1024, qc=256, gs=128, env={"FP6M_WK": 8, "FP6M_PAIR": pair}) for pair in (1, 0)]
        assert np.array_equal(outs[0].view(np.uint16), outs[1].view(np.uint16))
        run(oracle, m, 768, 512, qc=128, env={"FP6M_WK": 8, "FP6M_PAIR": 1})
    run(oracle, 30, 512, 512, qc=512, ksplit=2, env={"FP6M_WK": 8, "FP6M_PAIR": 1})
    run(oracle, 20, 256, 64, qc=-1, env={"FP6M_WK": 8, "FP6M_PAIR": 1})       # one k unit: idle slices
    run(oracle, 29, 1024, 8192, qc=256, gs=128)                           # the dispatcher's own choice of it
    for gs in (-1, 128):
        one_hot_case(oracle, 27, 768, 1024, 256, gs, {"wk": 8, "pair": 1})


def test_fp6_tiles_with_a_finer_k_split_than_int4_tiles(oracle):
    """m > 16 in a grid that is resident at once: the FP6 tiles' k range is cut into twice as many parts as the INT4
    tiles' (their own slice rule, divisor, partial-sum slots and counters); here 2 against 1 and 4 against 2, with
    group scales and without, ragged rows, both loops of the four-block kernel and the two-block one."""
    for pair in (1, 0):
        e = {"FP6M_PAIR": pair}
        run(oracle, 100, 512, 4096, qc=256, gs=128, sms=1, env=e)
        run(oracle, 100, 512, 2048, qc=256, sms=1, env=e)
        run(oracle, 70, 768, 8192, qc=384, gs=128, sms=2, env=e)
    run(oracle, 24, 512, 4096, qc=256, gs=128, sms=1)
    run(oracle, 130, 768, 4096, qc=256, sms=1, env={"FP6M_VERBOSE": 1})


def test_decode_kernel_with_eight_waves_per_workgroup(oracle):
    """The m <= 16 kernel with eight k slices per workgroup (picked for grids of about one workgroup per CU, e.g.
    8192 x 10240 at m = 1), forced on small and ragged problems, with and without a k split across workgroups."""
    e = {"FP6M_WK16": 8}
    for m in (1, 3, 4, 5, 16):
        run(oracle, m, 512, 1024, qc=256, gs=128, env=e)
        run(oracle, m, 768, 512, qc=128, env=e)
        run(oracle, m, 256, 64, 64, 256, qc=-1, env=e)                  # one k unit: seven idle waves
        run(oracle, m, 512, 2048, qc=256, ksplit=3, env=e)
    run(oracle, 1, 10240, 8192, qc=256, gs=128)                         # the dispatcher's own choice of it


def test_one_wave_decode_kernel(oracle):
    """The decode kernel (one wave per workgroup, every tile's k range cut into chunks that the waves draw from a
    counter, parts of a tile added into 64-bit cells): the dispatcher uses it for one row; here also forced for two to
    four rows, with few waves (every wave draws many chunks), as many waves as chunks (nothing to draw), chunks that
    do not divide a tile, whole tiles (sms = 1), FP6-only and INT4-only problems, both scale modes; and the
    workgroup kernel forced for one row."""
    for m in (1, 2, 3, 4):
        e = {"FP6M_SK": 1}
        run(oracle, m, 512, 2048, qc=256, gs=128, env=e)
        run(oracle, m, 512, 2048, qc=256, env=e)
        run(oracle, m, 768, 1024, qc=128, gs=128, env=dict(e, FP6M_SHARE=3))      # 8 units per tile: chunks of 3, 3, 2
        run(oracle, m, 768, 1024, qc=128, env=dict(e, FP6M_SHARE=5))              # 16 units per tile: 5, 5, 5, 1 -> 6, 6, 4
        run(oracle, m, 1024, 2048, qc=256, gs=128, env=dict(e, FP6M_WGS=7))       # seven waves for 150 chunks
        run(oracle, m, 1024, 2048, qc=256, gs=128, env=dict(e, FP6M_WGS=37, FP6M_SHARE=2))
        run(oracle, m, 1024, 2048, qc=256, env=dict(e, FP6M_WGS=100))
        run(oracle, m, 1024, 2048, qc=256, gs=128, env=dict(e, FP6M_WGS=100000))  # a wave per chunk
        run(oracle, m, 512, 2048, qc=256, gs=128, sms=1, env=e)                   # whole tiles, no cells
        run(oracle, m, 512, 2048, qc=256, gs=128, sms=1, env=dict(e, FP6M_WGS=3)) # ... drawn by three waves
        run(oracle, m, 512, 2048, qc=256, gs=128, sms=3, env=e)
        run(oracle, m, 512, 2048, qc=256, ksplit=16, env=e)
        run(oracle, m, 512, 1024, qc=512, env=e)                                  # all FP6
        run(oracle, m, 512, 1024, qc=512, env=dict(e, FP6M_WGS=5))
        run(oracle, m, 640, 1024, qc=-1, gs=128, env=dict(e, FP6M_SHARE=1))       # all INT4, one unit per chunk
        run(oracle, m, 768, 192, 64, 256, qc=-1, env=dict(e, FP6M_SHARE=2))       # three units per tile, no group scales
        run(oracle, m, 256, 64, 64, 256, qc=-1, env=e)                            # a single unit
        # k = 64 without group scales and fewer waves than tiles: an INT4 chunk of the single unit would be shorter than
        # the fetch side's look-ahead, which drawn chunks cannot follow, so the workgroup kernel takes these
        run(oracle, m, 1024, 64, 64, 256, qc=-1, env=dict(e, FP6M_WGS=3))
        run(oracle, m, 1024, 64, 64, 256, qc=256, env=dict(e, FP6M_WGS=3))
    run(oracle, 1, 512, 2048, qc=256, gs=128, env={"FP6M_SK": 0})                 # one row on the workgroup kernel
    run(oracle, 1, 768, 1024, qc=128, env={"FP6M_SK": 0})
    for gs in (-1, 128):
        one_hot_case(oracle, 4, 768, 1024, 256, gs, {"sk": 1, "share": 3, "wgs": 11})
        one_hot_case(oracle, 1, 768, 1024, 256, gs)
        one_hot_case(oracle, 1, 768, 1024, 256, gs, {"sk": 0})


def test_max_par_chunks_m(oracle):
    """m-tiles beyond max_par go to further launches (fp6_marlin_cuda_kernel.cu:917-948)."""
    run(oracle, 300, 512, 512, qc=256, max_par=2)
    run(oracle, 129, 256, 512, qc=-1, max_par=1)


def one_hot_case(oracle, m, n, k, qc, gs, knobs=None, max_par=16):
    """Row r of A is the unit vector e_(7r+3 mod k): row r of C must be row 7r+3 of the dequantised weight, bit for
    bit.  Exact in every kernel: per-column scales give fp16(q * s) from one fp32 product; group scales give the same
    value either as fp32(q) * fp32(s) rounded once (m <= 16) or as the fp16 product q * s formed before the MFMA
    (m > 16: fp16(q * s) is what the MFMA multiplies by 1.0); FP6 values have three significant bits, so value * s is
    exact in fp32 and rounded once."""
    import fp6_marlin
    print(f"case one-hot m={m} n={n} k={k} qc={qc} gs={gs} knobs={knobs}", flush=True)
    ref, B, s = problem(oracle, n, k, qc, gs, seed=3)
    hot = [(7 * r + 3) % k for r in range(m)]
    A = torch.zeros((m, k), dtype=torch.half)
    A[torch.arange(m), torch.tensor(hot)] = 1.0
    C = torch.full((m, n), float("nan"), dtype=torch.half, device=dev())
    ws = torch.zeros(n // 128 * 16, dtype=torch.int32, device=dev())
    with fp6_marlin.cabi.tuning(**(knobs or {})):
        fp6_marlin.mul(A.to(dev()), B, C, s, ws, qc, -1, -1, -1, max_par, gs)
        torch.cuda.synchronize()
    got = C.cpu().numpy().astype(np.float32)
    want = ref[hot].astype(np.float32)
    bad = np.argwhere(got != want)
    assert bad.size == 0, f"{len(bad)} wrong values, first at (row, col) {bad[0]}: {got[tuple(bad[0])]} != {want[tuple(bad[0])]}"
    assert int(ws.abs().sum().item()) == 0


def test_one_hot_rows_return_exact_weight_rows(oracle):
    """A = unit vectors: C must equal rows of the dequantised weight bit for bit (pins layout and scale order) --
    for the m <= 16 kernel, both loops of the m > 16 kernel, its two-block form and eight-wave form, with
    per-column and with group-128 scales."""
    shapes = [(512, 256, 256), (768, 1024, 256), (256, 512, 256), (640, 128, -1)]
    for n, k, qc in shapes:
        for gs in (-1, 128):
            if gs == 128 and k % 128:
                continue
            for m in (9, 16):                                           # gemm_m16_kernel, both ring widths
                one_hot_case(oracle, m, n, k, qc, gs)
    for n, k, qc in shapes[:2]:
        for gs in (-1, 128):
            one_hot_case(oracle, 24, n, k, qc, gs)                      # two 16-row blocks per wave
            one_hot_case(oracle, 40, n, k, qc, gs)                      # four blocks, ring loop
            one_hot_case(oracle, 100, n, k, qc, gs)                     # four blocks, paired loop (INT4 tiles)
            one_hot_case(oracle, 200, n, k, qc, gs, {"wk": 4})
            one_hot_case(oracle, 200, n, k, qc, gs, {"wk": 8})
            one_hot_case(oracle, 100, n, k, qc, gs, {"pair": 0})
            one_hot_case(oracle, 40, n, k, qc, gs, {"pair": 1})
            one_hot_case(oracle, 130, n, k, qc, gs, {"ksplit": 2})      # partial tiles through the scratch
            one_hot_case(oracle, 300, n, k, qc, gs, {"mb": 4})          # five 64-row tiles
            one_hot_case(oracle, 1100, n, k, qc, gs, {"pair": 1})


def test_baseline_config0(oracle):
    run(oracle, 16, 4096, 4096, qc=256, gs=128)


def test_baseline_config4_edge_shapes(oracle):
    import fp6_marlin
    # Llama-13B shapes, m=33, per-channel INT4, 512 FP6 columns.  Operands from the shipped packers
    # (bit-exact with the oracle, tests/test_cpu_routines.py); the oracle's literal prepacker is too slow here.
    for k, n in [(5120, 13824), (13824, 5120)]:
        print(f"case cfg4 k={k} n={n}", flush=True)
        g = torch.Generator().manual_seed(4)
        w = (torch.randn((k, n), generator=g) * 0.02).half()
        B, s, ref = fp6_marlin.pack_mixed_weight(w, 512, -1)
        A = torch.randn((33, k), generator=g).half()
        C = torch.full((33, n), float("nan"), dtype=torch.half, device=dev())
        ws = torch.zeros(n // 128 * 16, dtype=torch.int32, device=dev())
        fp6_marlin.mul(A.to(dev()), B.to(dev()), C, s.to(dev()), ws, 512)
        torch.cuda.synchronize()
        c_ref = (A.to(dev()).float() @ ref.to(dev()).float()).cpu().numpy()
        c = C.cpu().numpy()
        assert np.isfinite(c).all()
        err = oracle.rel_err(c, c_ref)
        assert err <= TOL, err
        for name, sl in (("INT4", slice(0, n - 512)), ("FP6", slice(n - 512, n))):     # each region alone, like `run`
            e = oracle.rel_err(c[:, sl], c_ref[:, sl])
            assert e <= TOL, f"rel err {e} on the {name} columns"
        assert int(ws.abs().sum().item()) == 0


LLAMA7B = [(4096, 12288), (4096, 4096), (4096, 22016), (11008, 4096)]
LLAMA70B = [(8192, 10240), (8192, 8192), (8192, 57344), (28672, 8192)]
MSWEEP = [1, 2, 4, 8, 16, 32, 64, 128, 256, 512, 1024]


def baseline_cases():
    """(k, n) -> row counts: every shape x M of the benchmark's Llama-2-7B, Llama-2-70B and M-sweep configurations, plus one
    launch of 1024 rows on a weight of 128 Mi elements, shapes that both workgroup kernels run with their INT4 tiles in two
    classes, and shapes picked for the other branches of the planners."""
    cases = {}
    for k, n in LLAMA7B:
        cases.setdefault((k, n), set()).update([1, 16])                 # config 1 (M = 1) and its M = 16 bench rows
    for k, n in LLAMA70B:
        cases.setdefault((k, n), set()).update([1, 16])                 # config 2
    cases[(8192, 8192)].update(MSWEEP)                                  # config 3
    cases.setdefault((8192, 16384), set()).add(1024)
    cases.setdefault((6656, 35328), set()).update([4, 16])              # a few more tiles than CUs: INT4 tiles in two classes
    cases.setdefault((8192, 36864), set()).update([32, 64])             # the same in the m > 16 kernel (32- and 64-row tiles)
    # shapes that take the planners' other branches: few tiles on a long k (eight-wave workgroups, at most eight parts; 40
    # chunks per tile at one row), splits that fit one workgroup per CU (eight waves, and four on a short k), a split no
    # finer than its longest slice needs, 256-row chunks at one row
    cases.setdefault((14336, 2048), set()).update([1, 8, 16, 32, 64])
    cases.setdefault((11008, 5120), set()).update([8, 48])
    cases.setdefault((5120, 15360), set()).update([6, 16])
    cases.setdefault((8192, 6144), set()).update([1, 32, 64])
    cases.setdefault((4096, 6144), set()).update([1, 4])
    return sorted((kn, sorted(ms)) for kn, ms in cases.items())


def tile_errors(c, ref, tile=128):
    """mean |c - ref| / mean |ref| of every 128-column tile (all rows)."""
    d = (c.float() - ref).abs().reshape(c.shape[0], -1, tile).mean(dim=(0, 2))
    r = ref.abs().reshape(c.shape[0], -1, tile).mean(dim=(0, 2))
    return d / r


@pytest.mark.parametrize("kn,ms", baseline_cases(), ids=lambda v: "x".join(map(str, v)) if isinstance(v, tuple) else None)
def test_baseline_full_sizes_against_unpacked_words(oracle, kn, ms):
    """The benchmark's Llama-2-7B, Llama-2-70B and M-sweep configurations at their real sizes, every shape x M.  The oracle cannot pack 8192 x 57344 in seconds, so
    the packed words are random bits (every FP6 code and INT4 nibble occurs) and the reference weight comes from the
    shipped unpacker, which tests/test_cpu_routines.py pins bit for bit against the oracle's dequantised weight; the
    reference product is an fp32 matmul of A with it.  The 1e-3 bar (test.py:181) is applied to every 128-column
    tile on its own, so an error confined to one tile or to the FP6 columns cannot hide in the mean over a wide
    matrix.  Also: two identical calls give identical bits, and linearity in A (C(a1 + a2) = C(a1) + C(a2))."""
    import fp6_marlin
    k, n = kn
    qc, gs = 256, 128
    g = torch.Generator().manual_seed(11 + k + n)
    n4 = n - qc
    words = k * n4 // 8 + k * qc * 3 // 16
    B = torch.randint(-2 ** 31, 2 ** 31 - 1, (words,), generator=g, dtype=torch.int64).to(torch.int32)
    s = (torch.rand((k // gs) * n4 + qc, generator=g) * 0.01 + 0.001).half()
    w = fp6_marlin.unpack_to_fp16(B, s, k, n, qc, gs).to(dev()).float()
    Bd, sd = B.to(dev()), s.to(dev())
    ws = torch.zeros(n // 128 * 16, dtype=torch.int32, device=dev())
    for m in ms:
        print(f"case full m={m} k={k} n={n}", flush=True)

        def gemm(a):
            C = torch.full((m, n), float("nan"), dtype=torch.half, device=dev())
            fp6_marlin.mul(a, Bd, C, sd, ws, qc, -1, -1, -1, 16, gs)
            torch.cuda.synchronize()
            return C

        a1 = torch.randn((m, k), generator=g).half().to(dev())
        c1 = gemm(a1)
        assert torch.equal(c1, gemm(a1)), (m, k, n, "two identical calls differ")
        ref = a1.float() @ w
        err = ((c1.float() - ref).abs().mean() / ref.abs().mean()).item()
        assert err <= TOL, (m, k, n, err)
        te = tile_errors(c1, ref)
        assert te.max().item() <= TOL, (m, k, n, "tile", int(te.argmax()), te.max().item())
        assert int(ws.abs().sum().item()) == 0
        # linearity: a2 is a small integer multiple pattern so that a1 + a2 is exact in fp16 for most entries
        a2 = (torch.randint(-2, 3, (m, k), generator=g).half() * 0.5).to(dev())
        a12 = (a1.float() + a2.float()).half()
        exact = (a12.float() == a1.float() + a2.float())
        a2 = torch.where(exact, a2, torch.zeros_like(a2))               # keep only entries whose sum is representable
        a12 = (a1.float() + a2.float()).half()
        lin = (gemm(a12).float() - (c1.float() + gemm(a2).float())).abs().mean() / ref.abs().mean()
        assert lin.item() <= TOL, (m, k, n, lin.item())
        del ref
    del w, Bd, sd
    torch.cuda.empty_cache()


def test_decode_chunk_lengths_by_generation(capfd):
    """One row on shapes whose chunk list exceeds the first generation of waves (4 x CUs): later generations get their
    own, shorter chunks (`gen2` / `gen3`: their waves' assumed share of a SIMD in per cent; `gen` = 0: equal chunks).
    Random words against the pinned unpacker, per 128-column tile, for the default and for forced ratios that send
    tiles to two and to three generations, with group scales and without; every setting twice, bit-identical; a
    column of A set to a unit vector returns the dequantised weight row exactly under every plan."""
    import fp6_marlin
    seen = set()
    for (k, n, qc, gs) in [(4096, 12288, 256, 128), (8192, 8192, 256, -1), (2048, 28672, 512, 128)]:
        g = torch.Generator().manual_seed(5 + k + n)
        n4 = n - qc
        B = torch.randint(-2 ** 31, 2 ** 31 - 1, (k * n4 // 8 + k * qc * 3 // 16,), generator=g, dtype=torch.int64).to(torch.int32)
        ns = (n4 if gs == -1 else (k // gs) * n4) + qc
        s = (torch.rand(ns, generator=g) * 0.01 + 0.001).half()
        w = fp6_marlin.unpack_to_fp16(B, s, k, n, qc, gs).to(dev())
        Bd, sd = B.to(dev()), s.to(dev())
        ws = torch.zeros(n // 128 * 16, dtype=torch.int32, device=dev())
        a = torch.randn((1, k), generator=g).half().to(dev())
        hot = torch.zeros((1, k), dtype=torch.half, device=dev())
        hot[0, k // 3] = 1.0
        ref = a.float() @ w.float()
        plans = set()
        for knobs in ({"gen": 0}, {}, {"gen2": 50, "gen3": 45}, {"gen2": 90, "gen3": 80}, {"gen2": 40, "gen3": 10}):
            print(f"case gen k={k} n={n} gs={gs} knobs={knobs}", flush=True)
            with fp6_marlin.cabi.tuning(verbose=1, **knobs):
                outs = []
                for rep in range(2):
                    C = torch.full((1, n), float("nan"), dtype=torch.half, device=dev())
                    fp6_marlin.mul(a, Bd, C, sd, ws, qc, -1, -1, -1, 16, gs)
                    torch.cuda.synchronize()
                    outs.append(C)
                plans.add(capfd.readouterr().err.strip().splitlines()[-1])
                assert torch.equal(outs[0], outs[1])
                te = tile_errors(outs[0], ref)
                assert te.max().item() <= TOL, (k, n, knobs, int(te.argmax()), te.max().item())
                C = torch.full((1, n), float("nan"), dtype=torch.half, device=dev())
                fp6_marlin.mul(hot, Bd, C, sd, ws, qc, -1, -1, -1, 16, gs)
                torch.cuda.synchronize()
                capfd.readouterr()
                assert torch.equal(C[0], w[k // 3]), (k, n, knobs)
        assert int(ws.abs().sum().item()) == 0
        assert len(plans) >= 2, plans                                    # the settings really led to different plans
        seen |= plans
        del w, Bd, sd
    import re
    assert any(re.search(r"by generation: \d+ tiles x \d+ chunks of \d+, [1-9]\d* x \d+ of \d+, 0 x", p) for p in seen), seen    # two generations
    assert any(re.search(r"by generation: \d+ tiles x \d+ chunks of \d+, [1-9]\d* x \d+ of \d+, [1-9]", p) for p in seen), seen  # three
    torch.cuda.empty_cache()


def test_layer_forward(oracle):
    import fp6_marlin
    torch.manual_seed(1)
    lin = torch.nn.Linear(1024, 768, bias=False).half()
    layer = fp6_marlin.Layer(1024, 768, groupsize=128, quant_cols=256)
    w_ref = layer.pack(lin)
    layer = layer.to(dev())
    x = torch.randn((2, 5, 1024), dtype=torch.half)
    y = layer(x.to(dev())).cpu()
    assert y.shape == (2, 5, 768)
    y_ref = (x.reshape(-1, 1024).float() @ w_ref.float()).reshape(2, 5, 768)
    assert oracle.rel_err(y.numpy(), y_ref.numpy()) <= TOL


def test_layer_forward_captured_in_a_hip_graph(oracle):
    """A Layer that has run once can be captured with torch.cuda.graph (whose capture stream is not the stream of the
    warm-up) and replayed: the default workspace belongs to the device, not to the stream.  Every replay, with eager
    forwards in between, gives the eager result bit for bit; a caller's own workspace works the same way."""
    import fp6_marlin
    k, n, m = 1024, 1536, 8
    rng = np.random.default_rng(11)
    lin = torch.nn.Linear(k, n, bias=False).half()
    lin.weight.data = torch.from_numpy(rng.normal(0, 0.02, (n, k)).astype(np.float16))
    layer = fp6_marlin.Layer(k, n, groupsize=128, quant_cols=256)
    w_ref = layer.pack(lin)
    layer = layer.to(dev())
    x = torch.from_numpy(rng.normal(0, 1, (m, k)).astype(np.float16)).to(dev())
    want = layer(x).clone()                                              # warm-up on the current stream
    assert oracle.rel_err(want.cpu().numpy(), oracle.matmul_ref(x.cpu().numpy(), w_ref.numpy())) <= TOL
    # (a workspace of the caller's own: given its region ahead of the capture, because by now the earlier tests'
    # workspaces hold every region, and a capture cannot wait for the device to take one over)
    own = fp6_marlin.init_workspace(torch.zeros(n // 128 * 16, dtype=torch.int32, device=dev()))
    for ws in (None, own):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y = layer(x, workspace=ws)
        for _ in range(3):
            y.fill_(float("nan"))
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y, want)
            assert torch.equal(layer(x, workspace=ws), want)             # eager work between the replays
    with pytest.raises(ValueError):
        layer(x, workspace=torch.zeros(8, dtype=torch.int32, device=dev()))
    fp6_marlin.release_workspace(own)


def test_layer_with_chosen_fp6_channels_bias_residual_and_checkpoint(oracle):
    """FP6 on arbitrary output features, results in the linear layer's own order, bias and residual in the call,
    both word orders; state_dict round trip and the refusal of a checkpoint of another format."""
    import fp6_marlin
    torch.manual_seed(2)
    k, n, qc = 512, 768, 128
    lin = torch.nn.Linear(k, n, bias=True).half()
    picked = torch.randperm(n)[:qc]
    x = torch.randn((3, 4, k), dtype=torch.half)
    res = torch.randn((3, 4, n), dtype=torch.half)
    outs = []
    for layout in ("reference", "gfx950"):
        layer = fp6_marlin.Layer(k, n, groupsize=128, quant_cols=qc, fp6_channels=picked, bias=True, layout=layout)
        w_ref = layer.pack(lin)
        # the check weight comes back in the linear layer's own column order (a wrong order would give ~1.4 here)
        err = (w_ref.float() - lin.weight.data.t().float()).abs().mean(0) / lin.weight.data.t().float().abs().mean(0)
        assert err.max() < 0.3
        layer = layer.to(dev())
        y = layer(x.to(dev()), residual=res.to(dev())).cpu()
        y_ref = (x.reshape(-1, k).float() @ w_ref.float() + lin.bias.data.float()).reshape(3, 4, n) + res.float()
        assert oracle.rel_err(y.numpy(), y_ref.numpy()) <= TOL
        outs.append(y)
        clone = fp6_marlin.Layer(k, n, groupsize=128, quant_cols=qc, fp6_channels=picked, bias=True, layout=layout)
        clone.load_state_dict(layer.state_dict())
        assert torch.equal(clone.to(dev())(x.to(dev()), residual=res.to(dev())).cpu(), y)
        other = fp6_marlin.Layer(k, n, groupsize=-1, quant_cols=qc, fp6_channels=picked, bias=True, layout=layout)
        with pytest.raises(RuntimeError, match="does not match"):
            other.load_state_dict(layer.state_dict())
    assert torch.equal(outs[0], outs[1])


def test_dispatcher_choices_over_many_shapes(oracle):
    """The dispatcher picks waves per workgroup and the k split per shape (rule + cost model): a sweep over decode
    shapes with random packed words against the pinned unpacker, so that every combination it can choose is exercised
    with real sizes (eight-wave workgroups without a k split, exact one- and two-per-CU grids, long k)."""
    import fp6_marlin
    g = torch.Generator().manual_seed(5)
    gs = 128
    for k, n, qc in [(1024, 2048, 256), (4096, 10240, 256), (4096, 17920, 256), (4096, 28672, 0), (4096, 32768, 256),
                     (5120, 5120, 256), (6656, 6656, 128), (6656, 17920, 256), (11008, 2048, 256), (13824, 5120, 512),
                     (8192, 28672, 256), (2048, 57344, 256)]:
        n4 = n - qc
        B = torch.randint(-2 ** 31, 2 ** 31 - 1, (k * n4 // 8 + k * qc * 3 // 16,), generator=g, dtype=torch.int64).to(torch.int32)
        s = (torch.rand((k // gs) * n4 + qc, generator=g) * 0.01 + 0.001).half()
        w = fp6_marlin.unpack_to_fp16(B, s, k, n, qc if qc else -1, gs).to(dev())
        Bd, sd = B.to(dev()), s.to(dev())
        ws = torch.zeros(n // 128 * 16, dtype=torch.int32, device=dev())
        for m in (1, 4, 16):
            print(f"case dispatch m={m} k={k} n={n} qc={qc}", flush=True)
            a = torch.randn((m, k), generator=g).half().to(dev())
            C = torch.full((m, n), float("nan"), dtype=torch.half, device=dev())
            fp6_marlin.mul(a, Bd, C, sd, ws, qc if qc else -1, -1, -1, -1, 16, gs)
            torch.cuda.synchronize()
            ref = a.float() @ w.float()
            err = ((C.float() - ref).abs().mean() / ref.abs().mean()).item()
            assert err <= TOL, (m, k, n, qc, err)
            assert int(ws.abs().sum().item()) == 0
        del w, Bd, sd
        torch.cuda.empty_cache()


def test_random_shapes_rows_and_limits_against_unpacked_words(oracle):
    """A seeded random walk over what the dispatcher can be asked: k and n in multiples of 256 (up to 8192 x 8192
    weights), any multiple of 128 FP6 columns including none and all, both scale modes, 1 .. 1500 rows, `max_par`
    16 .. 1 (several launches), `sms` limits.  Random packed words against the pinned unpacker and an fp32 matmul:
    the relative-error bar on each region, an element-wise bound so that nothing hides in a mean, C fully written,
    two calls bit-identical, the workspace left zero."""
    import random
    import fp6_marlin
    rnd = random.Random(11)
    g = torch.Generator().manual_seed(11)
    for ci in range(120):
        k = 256 * rnd.choice([1, 2, 3, 4, 6, 8, 11, 16, 20, 32])
        n = 256 * rnd.choice([1, 2, 3, 5, 8, 13, 16, 24, 32, 43, 64, 112])
        if k * n > 8192 * 8192:
            n = 2048
        qc = min(n, rnd.choice([0, 256, 256, 256, 512, n, 128, 384]))
        gs = rnd.choice([-1, 128])
        m = rnd.choice([rnd.randint(1, 16), rnd.randint(17, 64), rnd.randint(65, 300), rnd.randint(300, 1500), 64, 128, 129, 256, 1024])
        max_par = rnd.choice([16, 16, 16, 8, 2, 1])
        sms = rnd.choice([-1, -1, -1, 1, 2, 7, 64])
        n4 = n - qc
        B = torch.randint(-2 ** 31, 2 ** 31 - 1, (k * n4 // 8 + k * qc * 3 // 16,), generator=g, dtype=torch.int64).to(torch.int32)
        s = (torch.rand(((k // gs) * n4 if gs > 0 else n4) + qc, generator=g) * 0.01 + 0.001).half()
        qarg = qc if qc else -1
        print(f"case random {ci} m={m} k={k} n={n} qc={qc} gs={gs} max_par={max_par} sms={sms}", flush=True)
        w = fp6_marlin.unpack_to_fp16(B, s, k, n, qarg, gs).to(dev())
        Bd, sd = B.to(dev()), s.to(dev())
        ws = torch.zeros(n // 128 * max_par, dtype=torch.int32, device=dev())
        a = torch.randn((m, k), generator=g).half().to(dev())
        C = torch.full((m, n), float("nan"), dtype=torch.half, device=dev())
        C2 = torch.full_like(C, float("nan"))
        for out in (C, C2):
            fp6_marlin.mul(a, Bd, out, sd, ws, qarg, -1, -1, sms, max_par, gs)
            torch.cuda.synchronize()
        case = (ci, m, k, n, qc, gs, max_par, sms)
        assert torch.isfinite(C).all(), case
        assert torch.equal(C, C2), case
        assert int(ws.abs().sum().item()) == 0, case
        ref = a.float() @ w.float()
        for sl in (slice(0, n4), slice(n4, n)):
            if sl.stop > sl.start:
                r = ref[:, sl]
                d = (C[:, sl].float() - r).abs()
                assert (d.mean() / r.abs().mean()).item() <= TOL, case
                # fp16 rounding of the result plus the accumulation order: far below a wrong or missing k step
                assert bool((d <= 4e-3 * r.abs() + 0.13 * r.abs().mean()).all()), case
        del w, Bd, sd, a, C, C2, ref
        torch.cuda.empty_cache()


def test_long_k_with_a_poorly_filled_grid_takes_128_row_tiles_with_a_k_split(capfd):
    """13824 x 5120 at 256 rows: 160 workgroups of 64 rows would occupy 160 of 256 CUs with nothing left to split; the
    dispatcher takes 128-row tiles with three k parts instead (read back from its verbose output) and the result is
    checked per region against the pinned unpacker; on k = 8192 the rule does not apply."""
    import fp6_marlin
    g = torch.Generator().manual_seed(9)
    for k, n, want in ((13824, 5120, "MB=8 row tiles 2 ks4=3"), (8192, 5120, "MB=4")):
        qc, gs, m = 256, 128, 256
        n4 = n - qc
        B = torch.randint(-2 ** 31, 2 ** 31 - 1, (k * n4 // 8 + k * qc * 3 // 16,), generator=g, dtype=torch.int64).to(torch.int32)
        s = (torch.rand((k // gs) * n4 + qc, generator=g) * 0.01 + 0.001).half()
        w = fp6_marlin.unpack_to_fp16(B, s, k, n, qc, gs).to(dev())
        a = torch.randn((m, k), generator=g).half().to(dev())
        C = torch.full((m, n), float("nan"), dtype=torch.half, device=dev())
        ws = torch.zeros(n // 128 * 16, dtype=torch.int32, device=dev())
        capfd.readouterr()
        with fp6_marlin.cabi.tuning(verbose=1):
            fp6_marlin.mul(a, B.to(dev()), C, s.to(dev()), ws, qc, -1, -1, -1, 16, gs)
            torch.cuda.synchronize()
        err = capfd.readouterr().err
        assert want in err, (k, n, err[-300:])
        ref = a.float() @ w.float()
        for sl in (slice(0, n4), slice(n4, n)):
            d = (C[:, sl].float() - ref[:, sl]).abs()
            assert (d.mean() / ref[:, sl].abs().mean()).item() <= TOL
            assert bool((d <= 4e-3 * ref[:, sl].abs() + 0.13 * ref[:, sl].abs().mean()).all())
        assert int(ws.abs().sum().item()) == 0
