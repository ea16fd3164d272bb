"""The kernel choice (gemmlib_amd/csrc/blkq4_choose.h) and the launchers' dispatch agree, checked without a GPU
through blkq4_gemm_plan_sm80: for every shape the identity of the kernel the cost model picks equals the identity
of the kernel instantiation the launcher maps that choice to (a dry run: nothing is launched).

The reference's own choice is `m > 16` between two kernels (src/blkq4_f16_gemm_sm80.cu:343,
src/mickey/blk_q4/f16_gemm_sm80.h:63-72); the families below keep that much of it: GEMV and small batches stream
the weights (a few rows whose K a workgroup can request at once: the decode kernel), prefill shapes run MFMA tiles."""

import itertools

import pytest

MS = [1, 2, 4, 5, 8, 9, 16, 17, 24, 32, 33, 48, 64, 65, 96, 100, 128, 160, 200, 256, 300, 384, 512, 640, 768, 1000,
      1024, 1025, 1536, 2048, 3000, 4096, 8192]
NS = [32, 64, 256, 1024, 4096, 5120, 8192, 11008, 13824, 14336, 22016, 28672, 32000, 128256]
KS = [64, 128, 512, 1024, 2048, 4096, 5120, 8192, 11008, 14336, 28672]


def test_choice_equals_dispatch_over_a_sweep_of_shapes(capi):
    checked = 0
    kinds = set()
    for col, bf16 in itertools.product((True, False), (False, True)):
        for m, n, k in itertools.product(MS, NS, KS):
            if not col and n % 64:
                continue
            chosen, launched, text = capi.gemm_plan(64, col, m, n, k, has_offsets=(m + n + k) % 3 != 0, bf16=bf16)
            assert chosen == launched and chosen != 0, (col, bf16, m, n, k, hex(chosen), hex(launched), text)
            kinds.add(chosen)
            checked += 1
    assert checked > 15000 and len(kinds) >= 25  # many different kernels were asked for, every one of them exists


@pytest.mark.parametrize("bs", [16, 32, 64])
def test_every_block_size_has_every_kernel(capi, bs):
    for col in (True, False):
        for m, n, k in [(1, 4096, 4096), (16, 11008, 4096), (16, 28672, 8192), (1, 128256, 4096), (64, 4096, 4096),
                        (128, 4096, 4096), (256, 4096, 4096), (256, 4096, 11008), (768, 11008, 4096), (2048, 4096, 4096),
                        (4096, 28672, 8192), (32, 28672, 8192), (64, 28672, 4096), (1280, 14336, 8192)]:
            if not col and n % bs:
                continue
            chosen, launched, _ = capi.gemm_plan(bs, col, m, n, k)
            assert chosen == launched


def test_benchmark_configurations_get_the_expected_families(capi):
    plans = {name: capi.gemm_plan(bs, True, m, n, k, has_offsets=zp)[2] for name, (m, k, n, bs, zp) in {
        "C1": (64, 1024, 1024, 32, True), "C2": (1, 4096, 4096, 64, False), "C3": (16, 4096, 11008, 32, True),
        "C4": (2048, 4096, 4096, 64, True), "C5": (4096, 8192, 28672, 16, True)}.items()}
    assert plans["C2"] == "decode: 8 waves splitting K, 4 slices requested by each, 1 column tile(s) x 1 row(s), 256 workgroups"
    assert plans["C3"] == "decode: 8 waves splitting K, 4 slices requested by each, 3 column tile(s) x 16 row(s), 230 workgroups"
    assert plans["C1"].startswith("streaming:")
    assert plans["C4"].startswith("tile: 128 x 256, 4 + 4 waves, 256 tiles") and "parts" not in plans["C4"]
    assert plans["C5"].startswith("tile: 256 x 256, 4 + 0 waves, 1792 tiles") and "parts" not in plans["C5"]


def test_split_plans_are_well_formed(capi):
    import re
    seen = 0
    for m, n, k in itertools.product([65, 100, 128, 200, 256, 300, 512, 768, 1280], [2048, 4096, 5120, 8192, 11008, 14336, 28672],
                                     [1024, 4096, 5120, 8192, 11008, 14336, 28672]):
        text = capi.gemm_plan(64, True, m, n, k)[2]
        got = re.match(r"tile: (\d+) x (\d+), \d \+ \d waves, (\d+) tiles(?:, blocks of \d+ x \d+ tiles per XCD)?, the last (\d+) in (\d+) parts \(workspace (\d+) bytes\)", text)
        if not got:
            continue
        seen += 1
        bm, bn, tiles, split_tiles, parts, ws = map(int, got.groups())
        assert tiles == -(-m // bm) * -(-n // bn)
        assert split_tiles == (tiles % 256 or tiles) and 2 <= parts <= 4 and split_tiles * parts <= 256
        assert (k // 64) // parts >= 4                                     # every part has at least 4 k tiles
        assert ws == 16384 + split_tiles * parts * bm * bn * 4 <= 16384 + (32 << 20)
    assert seen > 50


def test_tile_order_in_blocks_per_xcd_is_well_formed(capi):
    """whole rounds of 256 tiles may be dealt to the 8 XCDs in blocks of rows x columns tiles: 32 tiles each, the rows a
    power of two that divides the problem's tile rows (the launcher's dry run has accepted every such plan)"""
    import re
    assert capi.gemm_plan(64, True, 512, 4096, 4096)[2] == "tile: 64 x 128, 4 + 4 waves, 256 tiles, blocks of 4 x 8 tiles per XCD"
    assert capi.gemm_plan(64, True, 2048, 4096, 4096)[2].endswith("blocks of 4 x 8 tiles per XCD")   # 0.8 of what 2 x 16 fetch
    assert "XCD" not in capi.gemm_plan(16, True, 4096, 28672, 8192)[2]     # 2 x 16 and 4 x 8 of its tiles fetch the same
    seen = 0
    for m, n, k in itertools.product([200, 256, 384, 512, 1024, 2048, 4096], [4096, 8192, 11008, 14336, 28672], [4096, 8192]):
        text = capi.gemm_plan(64, True, m, n, k)[2]
        got = re.match(r"tile: (\d+) x (\d+), \d \+ \d waves, (\d+) tiles, blocks of (\d+) x (\d+) tiles per XCD", text)
        if not got:
            continue
        seen += 1
        bm, bn, tiles, rows, cols = map(int, got.groups())
        m_tiles = -(-m // bm)
        assert rows * cols == 32 and m_tiles % rows == 0 and m_tiles & (m_tiles - 1) == 0 and tiles >= 256, text
    assert seen >= 5


def test_plan_rejects_what_the_gemm_rejects(capi):
    for args, message in [((48, True, 4, 64, 64), "Unsupported block size: 48"), ((32, True, 0, 64, 64), "Empty problem size: 0x64x64"),
                          ((32, True, 4, 64, 96), "Kernel execution failed: Error Invalid Problem"),
                          ((64, False, 4, 96, 64), "Kernel execution failed: Error Invalid Problem")]:
        with pytest.raises(capi.Blkq4Error) as e:
            capi.gemm_plan(*args)
        assert str(e.value) == message


@pytest.mark.parametrize("m", [1, 4, 16, 64, 2048])
def test_packed_weights_of_four_gib_and_more_are_refused_with_a_message(capi, m):
    """every kernel addresses the packed weights with 32-bit byte offsets: k * n / 2 stays below 4 GiB"""
    with pytest.raises(capi.Blkq4Error, match="must stay below 4 GiB"):
        capi.gemm_plan(64, True, m, 131072, 65536)   # exactly 4 GiB
    chosen, launched, text = capi.gemm_plan(64, True, m, 131072 - 32, 65536)
    assert chosen == launched and chosen != 0, text


def test_wide_layers_give_every_compute_unit_the_same_number_of_tiles(capi):
    """five to sixteen rows, rows staged per slice: 4 to 7 column tiles per workgroup, no more workgroups than one round
    of resident ones"""
    import re
    for m, k in ((16, 4096), (16, 8192), (8, 8192), (5, 11008), (4, 8192), (1, 11008)):
        for n in (13312, 14336, 18432, 22016, 24576, 28672):
            text = capi.gemm_plan(64, True, m, n, k)[2]
            if not text.startswith("streaming:") or "rows staged per slice" not in text:
                continue
            tiles_per_workgroup = int(re.search(r"(\d+) column tile", text).group(1))
            workgroups = int(re.search(r"(\d+) workgroups", text).group(1))
            assert 4 <= tiles_per_workgroup <= 7 and workgroups <= 256, (m, n, k, text)
            assert (n // 16 + tiles_per_workgroup - 1) // tiles_per_workgroup <= workgroups, (m, n, k, text)


def _plan_as_forced_text(text, m):
    """the plan text of blkq4_gemm_plan_sm80 -> the plan as blkq4_gemm_with_plan_sm80 takes it (None: not recognised)"""
    import re
    t = re.match(r"tile: (\d+) x (\d+), (\d+) \+ (\d+) waves( \(the computing waves split the k tile\))?, (\d+) tiles", text)
    if t:
        rows, cols, waves, pw = (int(t.group(i)) for i in (1, 2, 3, 4))
        parts = re.search(r" in (\d+) parts", text)
        blocks = re.search(r"blocks of (\d+) x (\d+) tiles per XCD", text)
        if t.group(5):
            key = f"tile {rows // 32} {cols // 32} 1 1 {pw} 4 1"
        else:
            key = f"tile {rows // 32} {cols // (32 * waves)} 1 {waves} {pw} 1 {parts.group(1) if parts else 1}"
        if blocks:
            key += f" {-(-m // rows) // int(blocks.group(1))}"   # row bands = tile rows / tile rows of a block
        return key
    s = re.match(r"streaming: (\d+) waves (splitting K|with column tiles of their own), (\d+) column tile\(s\) x (\d+) rows, "
                 r"(\d+) slices in flight, rows (staged per slice|whole in LDS)", text)
    if s:
        waves, nt, rows, depth = int(s.group(1)), int(s.group(3)), int(s.group(4)), int(s.group(5))
        return (f"streaming {depth} {nt} {rows // 16} {waves} {2 if s.group(6) == 'staged per slice' else 1} "
                f"{waves if s.group(2) == 'splitting K' else 1}")
    d = re.match(r"decode( \(blocks along N\))?: (\d+) waves splitting K, (\d+) slices requested by each, "
                 r"(\d+) column tile\(s\) x (\d+) row\(s\)", text)
    if d:
        return f"decode {d.group(5)} {d.group(4)} {d.group(2)} {d.group(3)}"
    return None


def test_chosen_plans_against_times_recorded_on_an_mi355x(capi):
    """The cost model against measurements, without a GPU: tests/golden/plan_times_mi355x.json holds, for 311 shapes
    (fp16 and bf16, blocks of 16 / 32 / 64, both blockings, M = 1 ... 2304 on the layers of 7B - 70B models, K from 1024), the measured
    time of every plan that exists for the shape (tests/golden/make_plan_times.py).  The plan the library chooses has to
    be within 5 % of the fastest recorded one for nine shapes in ten and never more than a fifth behind: a constant of
    blkq4_choose.h changed for the worse shows here.  (A plan the measurement did not force is skipped.)"""
    import json
    import os
    rows = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "plan_times_mi355x.json")))
    judged, behind, worst = 0, [], 1.0
    for r in rows:
        text = capi.gemm_plan(r["block_size"], r["column_wise"], r["m"], r["n"], r["k"], r["has_offsets"], r["bf16"])[2]
        key = _plan_as_forced_text(text, r["m"])
        assert key is not None, text
        if key not in r["us"] and " ".join(key.split()[:8]) in r["us"]:
            key = " ".join(key.split()[:8])   # (the same tiles in the plain order, where the order was not forced)
        fastest = min(r["us"].values())
        if key not in r["us"]:
            if key.startswith("streaming 4 2 1 8 2 8"):
                continue   # a streaming shape that the measurement does not force
            ratio = 1.6    # left out of the fixture: more than 1.6 times the fastest
        else:
            ratio = r["us"][key] / fastest
        judged += 1
        worst = max(worst, ratio)
        if ratio > 1.05:
            behind.append((r["bf16"], r["block_size"], r["column_wise"], r["m"], r["n"], r["k"], key, round(ratio, 3)))
    assert judged >= 300
    assert len(behind) <= judged // 10 and worst <= 1.2, behind
