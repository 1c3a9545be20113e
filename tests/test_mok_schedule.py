"""The MoK framework stage's schedule, enumerated on the CPU.

``pipelink_amd/stages/mok/framework/schedule.hpp`` is the code the kernel runs (tables of prefix sums, the eight
lists, item -> task); it is plain C++ on integers, so g++ compiles it here with the device markers defined away.
The checks are the properties the forward relies on (campaigns/mok/port/framework/interp_fwd.cu:137-214 is the
reference's task decode): every tile of each GEMM is in exactly one list, exactly once; a tile's rows and columns
are the ones its number says; in a launch of both GEMMs every list holds its gate/up tiles in front of its down tiles
and a down tile waits for the counter of its own row tile; the search's cursor is a hint and nothing more.
"""
import os
import random
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FRAMEWORK = os.path.join(ROOT, "pipelink_amd", "stages", "mok", "framework")

GATE_UP, DOWN, BOTH = 3, 5, 0
TILE_X = 256

HARNESS = r"""
#define MOK_SCHED_FN inline
#define MOK_SCHED_UNIFORM(x) (x)
#include "schedule.hpp"
#include <cstdio>
#include <cstdlib>
#include <vector>
using namespace mok_framework;
static bool same(const MokGemmTask& a, const MokGemmTask& b) {
  return a.op == b.op && a.expert == b.expert && a.row_begin == b.row_begin && a.row_end == b.row_end &&
         a.col_begin == b.col_begin && a.task_idx == b.task_idx && a.counter_idx == b.counter_idx &&
         a.wait_target == b.wait_target && a.flags == b.flags;
}
int main(int argc, char** argv) {
  const int op = atoi(argv[1]), gu = atoi(argv[2]), dn = atoi(argv[3]);
  std::vector<int32_t> counts;
  for (int a = 4; a < argc; ++a) counts.push_back(atoi(argv[a]));
  const int ne = (int)counts.size();
  static Tables tab;
  tab.fill(counts.data(), ne);
  const MokFrameworkParams g{counts.data(), nullptr, ne, op, gu, dn};
  const Schedule sched{g, tab, tab.tile_begin[ne], op == MOK_GEMM_FWD_ROUTED_DOWN ? 0 : gu, op == MOK_GEMM_FWD_ROUTED_GATE_UP ? 0 : dn};
  printf("tiles %d rows %d\n", tab.tile_begin[ne], tab.row_begin[ne]);
  for (int q = 0; q < NUM_XCD; ++q) {
    const int n = sched.length(q);
    int cursor = 0;
    for (int i = 0; i < n; ++i) {
      const MokGemmTask t = sched.decode(q, i, cursor);
      // the cursor is only a place to start the search from: any expert gives the same task
      for (int hint = 0; hint < ne; hint += (ne > 8 ? ne / 8 : 1)) {
        int c = hint;
        if (!same(t, sched.decode(q, i, c)) || c != cursor) { printf("cursor %d changes item %d of list %d\n", hint, i, q); return 2; }
      }
      printf("%d %d %d %d %d %d %d %d %d\n", q, i, t.op, t.expert, t.row_begin, t.row_end, t.col_begin, t.counter_idx, t.wait_target);
    }
  }
  return 0;
}
"""


@pytest.fixture(scope="module")
def enumerate_schedule(tmp_path_factory):
    if shutil.which("g++") is None:
        pytest.skip("needs g++")
    d = tmp_path_factory.mktemp("mok_schedule")
    src = d / "enumerate.cpp"
    src.write_text(HARNESS)
    exe = d / "enumerate"
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Werror", f"-I{FRAMEWORK}", str(src), "-o", str(exe)], check=True)

    def run(op, gu, dn, counts):
        out = subprocess.run([str(exe), str(op), str(gu), str(dn), *map(str, counts)], check=True, capture_output=True, text=True).stdout
        lines = out.splitlines()
        head = lines[0].split()
        items = [tuple(map(int, line.split())) for line in lines[1:]]
        return int(head[1]), int(head[3]), items

    return run


def check(op, gu, dn, counts, tiles, rows, items):
    row_start = [0]
    for c in counts:
        row_start.append(row_start[-1] + c)
    tile_start = [0]
    for c in counts:
        tile_start.append(tile_start[-1] + (c + TILE_X - 1) // TILE_X)
    assert tiles == tile_start[-1] and rows == row_start[-1]
    run_gu, run_dn = op != DOWN, op != GATE_UP
    expected = set()
    for e, c in enumerate(counts):
        for r in range((c + TILE_X - 1) // TILE_X):
            if run_gu:
                expected |= {(GATE_UP, e, r, col) for col in range(gu)}
            if run_dn:
                expected |= {(DOWN, e, r, col) for col in range(dn)}
    seen = set()
    per_list = {}
    for q, i, top, e, row_begin, row_end, col_begin, counter_idx, wait_target in items:
        assert top in (GATE_UP, DOWN)
        width = 128 if top == GATE_UP else 256
        assert col_begin % width == 0
        local = row_begin - row_start[e]
        assert local >= 0 and local % TILE_X == 0 and row_begin < row_end == row_start[e + 1]
        key = (top, e, local // TILE_X, col_begin // width)
        assert key not in seen, f"tile {key} handed out twice"
        seen.add(key)
        if op == BOTH:
            assert counter_idx == tile_start[e] + local // TILE_X
        else:
            assert counter_idx == -1
        assert wait_target == (gu if top == DOWN and op == BOTH else 0)  # a GEMM launched alone waits for nothing
        per_list.setdefault(q, []).append((i, top))
    assert seen == expected
    total = len(expected)
    for q, entries in per_list.items():
        assert [i for i, _ in entries] == list(range(len(entries)))
        ops = [top for _, top in entries]
        assert ops == sorted(ops), f"list {q}: a down tile in front of a gate/up tile"  # GATE_UP (3) < DOWN (5)
        assert abs(len(entries) - total / 8) <= 2  # each GEMM's tiles are cut into eighths by number
    assert sum(len(v) for v in per_list.values()) == total


CASES = [
    (BOTH, 23, 12, [1024] * 32),
    (BOTH, 23, 12, [1037, 980, 1, 0, 256, 257, 255, 512, 3000, 0, 0, 64, 65]),
    (BOTH, 1, 1, [5]),
    (BOTH, 3, 2, [0, 0, 0, 300, 0]),
    (GATE_UP, 23, 12, [700, 1, 1, 1, 1, 1, 1, 1, 1, 900]),
    (DOWN, 23, 12, [700, 1, 1, 1, 1, 1, 1, 1, 1, 900]),
    (BOTH, 2, 1, [1] * 256),
    (BOTH, 23, 12, [0, 0, 0]),
]


@pytest.mark.parametrize("op,gu,dn,counts", CASES)
def test_every_tile_is_in_exactly_one_list_once(enumerate_schedule, op, gu, dn, counts):
    tiles, rows, items = enumerate_schedule(op, gu, dn, counts)
    check(op, gu, dn, counts, tiles, rows, items)


def test_random_expert_histograms(enumerate_schedule):
    rng = random.Random(20240607)
    for _ in range(25):
        ne = rng.choice([1, 2, 7, 8, 9, 32, 33, 128])
        counts = [rng.choice([0, 0, 1, 63, 64, 65, 255, 256, 257, rng.randrange(0, 1500)]) for _ in range(ne)]
        gu, dn = rng.choice([(23, 12), (1, 1), (4, 2), (2, 5)])
        op = rng.choice([BOTH, BOTH, GATE_UP, DOWN])
        tiles, rows, items = enumerate_schedule(op, gu, dn, counts)
        check(op, gu, dn, counts, tiles, rows, items)


def test_the_benchmark_histogram_has_the_tile_counts_the_design_quotes(enumerate_schedule):
    import json
    fixture = os.path.join(ROOT, "tests", "golden", "routing_seed0_T8192_E32_top4.json")
    if not os.path.exists(fixture):
        pytest.skip("routing fixture not present")
    counts = json.load(open(fixture))["tokens_per_expert"]
    tiles, rows, items = enumerate_schedule(BOTH, 23, 12, counts)
    check(BOTH, 23, 12, counts, tiles, rows, items)
    assert rows == 32768 and tiles == 143 and len(items) == 5005
    few_rows = sum(1 for it in items if it[5] - it[4] <= 64)
    assert few_rows == 15 * 35
