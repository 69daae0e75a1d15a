"""The index maps and the host walk of the kernel's decomposition (intra_amd/csrc/intra_maps.h)
compiled with g++ -fsanitize=address,undefined and run over ragged, tiny and ordinary shapes of all
seven maps: an out-of-range token position writes outside the exact S*S count array (a heap
overflow for AddressSanitizer), a signed overflow or a bad shift in the index arithmetic stops
UndefinedBehaviorSanitizer.  The program also requires every score to be computed at most once and
prints the pairs it counted, which the test compares with the oracle's masks.  The GPU runs the
same maps; sanitizers exist for the host only."""
import os
import shutil
import subprocess

import pytest

import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

SRC = r"""
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <vector>
#include "intra_maps.h"

static IntraGeom geom(int S) {
  IntraGeom ge;
  memset(&ge, 0, sizeof ge);
  ge.S = S; ge.G = 1; ge.window = 64; ge.width = 16; ge.text_len = 8; ge.pg = 1; ge.tm = 1; ge.blk = 64;
  ge.sink_chunk = 1024;
  return ge;
}

static int g_waves = 8;  // wavefronts per workgroup of the walks

// tiles whose key positions a map calls affine (tile_rows): every key where the formula puts it
template <class MAP>
static void check_tile_rows(const IntraGeom& ge, int pos) {
  const int n_sets = MAP::num_sets(ge);
  for (int set = 0; set < n_sets; ++set) {
    const int nq = MAP(ge, set, 0).nq();
    for (int t0 = 0; t0 < nq; t0 += pos) {
      const MAP map(ge, set, t0);
      const int kt_lo = MAP::kHasPrefix ? 0 : map.klo(t0);
      for (int t_first = kt_lo; t_first < map.nk() + 64; t_first += 64) {
        TileRows tr;
        if (!map_tile_rows(map, t_first, tr)) continue;
        for (int g = 0; g < 16; ++g)
          for (int r = 0; r < 4; ++r)
            if (t_first + 4 * g + r >= map.nk() || tr.base + g * tr.group_step + r * tr.row_step != map.kpos(t_first + 4 * g + r)) {
              printf("tile_rows differs from kpos: set %d t0 %d tile %d key %d\n", set, t0, t_first, 4 * g + r);
              exit(3);
            }
      }
    }
  }
}

template <class MAP>
static long walk(IntraGeom ge, int hp) {
  geom_finish(ge);
  check_tile_rows<MAP>(ge, g_waves * 32 / hp);
  std::vector<uint8_t> count((size_t)ge.S * ge.S, 0);  // exact size: a position >= S lands in a redzone
  im_model_walk<MAP>(ge, hp, g_waves, 64, count.data());
  long pairs = 0;
  for (uint8_t c : count) {
    if (c > 1) { printf("a score was computed %d times\n", (int)c); exit(2); }
    pairs += c;
  }
  return pairs;
}

int main() {
  const int hps[] = {1, 2, 4};
  for (int waves : {8, 4})
  for (int hp : hps) {
    g_waves = waves;
    for (int S : {1, 5, 63, 64, 65, 257, 777, 1000, 2048}) {
      for (int G : {1, 2, 3, 8, 13}) { IntraGeom ge = geom(S); ge.G = G; printf("scatter %d %d %d %ld\n", hp, S, G, walk<MapLlmScatter>(ge, hp)); }
      for (int G : {2, 8}) { IntraGeom ge = geom(S); ge.G = G; printf("gather1 %d %d %d %ld\n", hp, S, G, walk<MapLlmGather1>(ge, hp)); }
      for (int W : {64, 65, 130, 576, 5000}) { IntraGeom ge = geom(S); ge.window = W; printf("window %d %d %d %ld\n", hp, S, W, walk<MapLlmWindow>(ge, hp)); }
      for (int W : {1, 2, 63, 575}) for (int ns : {0, 1, 64, 700}) {
        IntraGeom ge = geom(S); ge.window = W; ge.ns = ns;
        printf("window_sink %d %d %d %d %ld\n", hp, S, W, ns, walk<MapLlmWindowSink>(ge, hp));
      }
      for (int G : {1, 2, 3}) for (int off = 0; off < G; ++off) for (int ns : {0, 1, 64}) {
        const int blk = off != 0 ? 256 : 64;  // a stripe offset keeps row blocks inside a query block
        IntraGeom ge = geom(S); ge.G = G; ge.blk = blk; ge.off = off; ge.ns = ns;
        printf("block_scatter %d %d %d %d %d %d %ld\n", hp, S, G, blk, off, ns, walk<MapLlmBlockScatter>(ge, hp));
      }
    }
    for (int width : {16, 24, 40}) for (int text : {8, 72, 128, 200}) {
      IntraGeom ge = geom(text + width * width); ge.width = width; ge.text_len = text;
      printf("image_scatter %d %d %d %ld\n", hp, width, text, walk<MapImgScatter>(ge, hp));
      int pg = waves * 32 / hp / 64;
      if (pg < 1) continue;  // (a row block holds whole patches)
      while ((width / 8) % pg != 0) --pg;
      for (int tm : {1, 2}) {
        const int chunk = text / 8;
        if (tm == 2 && (chunk % 32 != 0 || 2 * chunk > waves * 32 / hp)) continue;  // what the launcher allows
        ge.pg = pg; ge.tm = tm;
        printf("image_gather0 %d %d %d %ld\n", hp, width, text, walk<MapImgGather0F>(ge, hp));
      }
    }
  }
  g_waves = 8;
  { IntraGeom ge = geom(512 + 32 * 32); ge.width = 32; ge.text_len = 512; ge.pg = 4; ge.tm = 2;
    printf("image_gather0 1 32 512 %ld\n", walk<MapImgGather0F>(ge, 1)); }
  g_waves = 4;
  { IntraGeom ge = geom(512 + 32 * 32); ge.width = 32; ge.text_len = 512; ge.pg = 2; ge.tm = 1;
    printf("image_gather0 1 32 512 %ld\n", walk<MapImgGather0F>(ge, 1)); }
  printf("done\n");
  return 0;
}
"""


def expected_pairs(fields):
    kind, nums = fields[0], [int(x) for x in fields[1:-1]]
    if kind == "scatter":
        return int(oracle.llm_scatter_mask(nums[1], nums[2]).sum())
    if kind == "gather1":
        return int(oracle.llm_gather1_mask(nums[1], nums[2]).sum())
    if kind == "window":
        return int(oracle.llm_window_mask(nums[1], nums[2]).sum())
    if kind == "window_sink":
        return int(oracle.llm_window_sink_mask(nums[1], nums[2], nums[3]).sum())
    if kind == "block_scatter":
        return int(oracle.llm_block_scatter_mask(nums[1], nums[2], nums[3], nums[4], nums[5]).sum())
    width, text = nums[1], nums[2]
    return int(oracle.mask_rows("image/" + kind.split("_")[1], text + width * width, width=width, text_len=text).sum())


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_index_maps_and_host_walk_under_address_and_ub_sanitizers(tmp_path):
    src = tmp_path / "walk_san.cpp"
    src.write_text(SRC)
    exe = tmp_path / "walk_san"
    subprocess.run(["g++", "-O1", "-g", "-std=c++17", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
                    "-I", os.path.join(ROOT, "intra_amd", "csrc"), str(src), "-o", str(exe)], check=True)
    env = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=0", UBSAN_OPTIONS="print_stacktrace=1")
    res = subprocess.run([str(exe)], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, env=env, timeout=900)
    assert res.returncode == 0, (res.stdout[-2000:], res.stderr[-4000:])
    lines = res.stdout.strip().splitlines()
    assert lines[-1] == "done" and len(lines) > 500
    # the pair counts of a sample of the shapes against the oracle's masks (all of them would take minutes)
    for line in lines[:-1][::7]:
        fields = line.split()
        assert int(fields[-1]) == expected_pairs(fields), line
