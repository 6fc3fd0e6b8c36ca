"""The launch shapes the kernels were given, measured against their alternatives
on the device the test runs on (tests/native/launch_shapes.hip).  Fails when a
shape the library uses has fallen more than 12 % behind the best alternative, or
when the two workgroup numberings of the strided reduce disagree."""
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
SLACK = 1.12


@pytest.fixture(scope="module")
def table(gpu):
    exe = os.path.join(HERE, "native", "launch_shapes")
    assert os.path.exists(exe), "tests/native/launch_shapes is not built; run `python -m tests.native.build`"
    out = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    print(out.stdout)
    assert out.returncode == 0, out.stdout
    return out.stdout


def stream_rows(table):
    rows = {}
    for line in table.splitlines():
        m = re.match(r"stream (\w+)\s+(\d+) MB:(.*)", line)
        if m:
            rows[(m.group(1), int(m.group(2)))] = {k: float(v) for k, v in re.findall(r"(\S+x\d) (\d+\.\d+)", m.group(3))}
    return rows


# what the library launches: elementwise kernels single waves with one vector per lane,
# Blas::Set 256 lanes, the read probe of the harness 1024 lanes
USED = {"copy": "T64x1", "write": "T256x1", "read": "T1024x1"}


@pytest.mark.parametrize("kind", ["copy", "read", "write"])
@pytest.mark.parametrize("mb", [51, 411])
def test_stream_shape_in_use_is_among_the_fastest(table, kind, mb):
    row = stream_rows(table)[(kind, mb)]
    assert len(row) == 10
    best = min(row.values())
    assert row[USED[kind]] <= SLACK * best, (kind, mb, USED[kind], row)


def test_single_wave_workgroups_cap_one_directional_streams(table):
    """Why Set and the reductions do not use them: a wave that moves 1 KB is over too soon."""
    rows = stream_rows(table)
    for kind in ("read", "write"):
        assert rows[(kind, 411)]["T64x1"] > 1.2 * rows[(kind, 411)]["T256x1"]


def test_xcd_contiguous_numbering_of_the_strided_reduce(table):
    rows = re.findall(r"strided L(\d+)\s+(\S+)\s+(\d+\.\d+) (\w+)", table)
    assert len(rows) == 6 and all(r[3] == "same" for r in rows)
    t = {(int(l), kind): float(us) for l, kind, us, _ in rows}
    assert t[(32, "xcd-contiguous")] <= SLACK * min(t.values())
    assert t[(32, "xcd-contiguous")] <= 1.02 * t[(32, "round-robin")]


def tile_rows(table):
    flat, rows = {}, {}
    for line in table.splitlines():
        m = re.match(r"tile \[(\d+),(\d+),(\d+)\] flat (\d+\.\d+)", line)
        if m:
            flat[int(m.group(3))] = float(m.group(4))
        m = re.match(r"tile \[(\d+),(\d+),(\d+)\] (T\d+x\d+) (\w+)\s+(\w+)\s+(\d+\.\d+) (\w+)", line)
        if m:
            assert m.group(8) == "same", line
            rows[(int(m.group(3)), m.group(4), m.group(5), m.group(6))] = float(m.group(7))
    return flat, rows


def test_channel_tile_shape_in_use_and_what_the_pattern_costs(table):
    """The channel-tile kernels use 256 lanes, streaming stores where the rows start on
    64-byte boundaries and plain ones elsewhere, and park the tile in LDS.  As a pure
    copy that shape is within the slack of the alternatives, LDS and barriers included,
    and the pattern itself stays well behind a flat copy of the same bytes: that, not
    the folds, bounds those kernels."""
    flat, rows = tile_rows(table)
    assert len(rows) == 13
    for inner, used in ((3136, ("T256x16", "streaming", "parked")), (1444, ("T256x16", "plain", "parked"))):
        mine = {k[1:]: v for k, v in rows.items() if k[0] == inner}
        assert mine[used] <= SLACK * min(mine.values()), (inner, mine)
        assert min(mine.values()) > 1.10 * flat[inner], (inner, flat[inner], mine)


def test_a_lone_chain_of_ordered_additions_is_bound_by_latency(table):
    """The in-order sums (whole-plane average, Softmax, Normalize) are one dependent chain per row or column:
    a chain alone on its SIMD pays the latency of every addition, several waves (or chains) per SIMD share it.
    The kernels' rows-per-wave choices rest on these figures."""
    rows = {(int(w), int(c)): (float(a), float(b))
            for w, c, a, b in re.findall(r"add chain waves (\d+) chains (\d+): (\d+\.\d+) (\d+\.\d+)", table)}
    assert len(rows) == 7
    lone_chain, _ = rows[(1, 1)]
    _, simd_rate = rows[(8, 1)]
    assert lone_chain > 2.0 * simd_rate, rows  # one chain leaves most of the SIMD's issue slots empty
    assert rows[(1, 4)][1] < lone_chain, rows   # chains interleaved inside one wave share the latency too
