"""Result checks of the launch-shape probe (tests/native/launch_shapes.hip): every
alternative numbering of the strided reduce and every variant of the channel-tile
copy has to produce the same bits as the shape the library uses.  The probe also
prints timings; comparing those is `python bench.py --launch-shapes`, a
measurement, and no part of this suite."""
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def table(gpu):
    exe = os.path.join(HERE, "native", "launch_shapes")
    assert os.path.exists(exe), "tests/native/launch_shapes is not built; run `python -m tests.native.build`"
    out = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    print(out.stdout)
    assert out.returncode == 0, out.stdout
    return out.stdout


def test_every_table_of_the_probe_is_there(table):
    assert len(re.findall(r"^stream (\w+)\s+(\d+) MB:", table, re.M)) == 6
    assert len(re.findall(r"^add chain waves (\d+) chains (\d+):", table, re.M)) == 7
    assert "DIFFERENT" not in table
    assert "numberings same" in table  # xcd_contiguous and xcd_runs visit every work item once, grids of 1 to 3000


def test_both_numberings_of_the_strided_reduce_give_the_same_maxima(table):
    rows = re.findall(r"strided L(\d+)\s+(\S+)\s+(\d+\.\d+) (\w+)", table)
    assert len(rows) == 6 and all(r[3] == "same" for r in rows), rows


def test_every_channel_tile_variant_copies_the_tensor_unchanged(table):
    rows = re.findall(r"tile \[\d+,\d+,\d+\] T\d+x\d+ \w+\s+\w+\s+\d+\.\d+ (\w+)", table)
    assert len(rows) == 13 and all(r == "same" for r in rows), rows


def test_the_single_launch_sums_agree_with_the_two_launches(table):
    rows = re.findall(r"^full sum (two launches|ticket)[^\n]*? (\d+\.\d+) (\w+)$", table, re.M)
    assert len(rows) == 5 and all(r[2] == "same" for r in rows), rows
