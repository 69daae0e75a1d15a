"""The multiply-high division used by the index maps and by the kernel's work-item location,
checked on the host against integer division (compiled with g++ from the same header)."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

SRC = r"""
#include <stdio.h>
#include <stdlib.h>
#include <initializer_list>
#include "intra_maps.h"
int main() {
  long bad = 0, n_checked = 0;
  unsigned seed = 12345;
  for (int d = 1; d <= 70000; d += (d < 5000 ? 1 : 37)) {
    FastDiv f = make_fastdiv(d);
    for (int i = 0; i < 400; ++i) {
      unsigned n;
      if (i < 100) n = (unsigned)i;
      else if (i < 200) n = (unsigned)((long long)d * (i - 100) + (i & 1 ? d - 1 : 0)) & 0x7fffffffu;
      else if (i < 210) n = 0x7fffffffu - (unsigned)(i - 200);
      else { seed = seed * 1664525u + 1013904223u; n = seed >> 1; }
      ++n_checked;
      if (fd_div(n, f) != n / (unsigned)d || fd_mod(n, f) != n % (unsigned)d) {
        if (bad++ < 5) printf("mismatch n=%u d=%d got %u\n", n, d, fd_div(n, f));
      }
    }
  }
  int big[] = {1 << 20, (1 << 20) + 1, 1 << 30, (1 << 30) + 12345, 0x7fffffff};
  for (int d : big) {
    FastDiv f = make_fastdiv(d);
    for (unsigned n : {0u, 1u, (unsigned)d - 1, (unsigned)d, 0x7ffffffeu, 0x7fffffffu}) {
      ++n_checked;
      if (fd_div(n, f) != n / (unsigned)d) { ++bad; printf("mismatch n=%u d=%d\n", n, d); }
    }
  }
  printf("checked %ld bad %ld\n", n_checked, bad);
  return bad != 0;
}
"""


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_fastdiv_matches_integer_division(tmp_path):
    src = tmp_path / "fastdiv_check.cpp"
    src.write_text(SRC)
    exe = tmp_path / "fastdiv_check"
    subprocess.run(["g++", "-O1", "-std=c++17", "-I", os.path.join(ROOT, "intra_amd", "csrc"), str(src), "-o", str(exe)],
                   check=True)
    res = subprocess.run([str(exe)], stdout=subprocess.PIPE, text=True)
    assert res.returncode == 0, res.stdout
