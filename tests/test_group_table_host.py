"""The grouped GEMM's M tile table on the CPU: the builder's and the tile walk's own arithmetic
(wave_amd/csrc/mxfp4_group_table.h, compiled for the host by tests/host_group_table.cpp) over well-formed and
malformed offsets arrays, with and without short tiles.  Every tile the walk reaches must be an entry the builder
wrote, with its rows inside the tensors, its group below the group count, every (M tile, N tile) visited exactly
once, and every short tile (a group's last tile of few rows) behind all full ones.

The reference's MoE tests build their groups from torch.unique counts and never hand over a malformed array
(tests/kernel/moe_test.py:175-246); a C ABI that takes a device pointer has to survive one.
"""

import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def harness(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("grp") / "host_group_table")
    subprocess.check_call(["g++", "-O1", "-std=c++17", "-Wall", "-fsanitize=address,undefined", "-o", exe,
                           os.path.join(ROOT, "tests", "host_group_table.cpp")])
    return exe


def run(harness, cases):
    text = "".join(f"{t} {bm} {tn} {sr} {len(off) - 1} {' '.join(str(int(o)) for o in off)}\n" for t, bm, tn, sr, off in cases)
    out = subprocess.run([harness], input=text, capture_output=True, text=True)
    assert out.returncode == 0, out.stderr[-2000:]
    lines = out.stdout.split("\n")[:-1]
    assert len(lines) == len(cases)
    return lines


def test_well_formed_offsets_make_every_tile(harness):
    rng = np.random.default_rng(0)
    cases = []
    for _ in range(300):
        groups = int(rng.integers(1, 40))
        bm = int(rng.choice([128, 256]))
        counts = rng.multinomial(int(rng.integers(0, 9000)), np.ones(groups) / groups)
        if rng.random() < 0.3:
            counts[rng.integers(0, groups)] = 0
        off = np.concatenate([[0], np.cumsum(counts)])
        cases.append((int(off[-1]) + int(rng.integers(0, 300)), bm, int(rng.integers(1, 60)), int(rng.choice([0, 64, 128])), off))
    for (t, bm, tn, sr, off), line in zip(cases, run(harness, cases)):
        counts = [int(c) for c in np.diff(off)]
        shorts = sum(1 for c in counts if c > 0 and c - (-(-c // bm) - 1) * bm <= sr)
        assert line == f"ok {sum(-(-c // bm) for c in counts)} {shorts}", (t, bm, tn, sr, off.tolist(), line)


def test_the_capacity_cut_keeps_the_walk_inside_the_table(harness):
    # the advisor's example: [0, T, 0, T, ...] with T = 2560 and 8 groups is 40 tiles against a capacity of 18
    T = 2560
    cases = [(T, 256, 7, 0, [0, T] * 4 + [0]), (T, 256, 56, 64, [0, T, 0, T, 0, T, 0, T, T]),
             (T + 40, 256, 5, 64, [0, T + 40] * 4 + [0])]
    rng = np.random.default_rng(1)
    for _ in range(2000):
        groups = int(rng.integers(1, 24))
        total = int(rng.integers(0, 6000))
        kind = rng.integers(0, 4)
        if kind == 0:  # anything at all, negative and beyond the tensor included
            off = rng.integers(-3000, 2 * total + 3000, groups + 1)
        elif kind == 1:  # every group is most of the tensor
            off = np.where(np.arange(groups + 1) % 2 == 0, 0, total)
        elif kind == 2:  # sorted but not starting at 0 / ending at total
            off = np.sort(rng.integers(0, total + 1, groups + 1))
        else:  # a well-formed array with two entries swapped
            off = np.sort(rng.integers(0, total + 1, groups + 1))
            i, j = rng.integers(0, groups + 1, 2)
            off[i], off[j] = off[j], off[i]
        cases.append((total, int(rng.choice([64, 128, 256])), int(rng.integers(1, 20)), int(rng.choice([0, 16, 64])), off))
    bad = [(c[0], c[1], c[2], c[3], list(map(int, c[4])), line) for c, line in zip(cases, run(harness, cases)) if not line.startswith("ok")]
    assert not bad, bad[:3]
