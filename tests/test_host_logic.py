"""Host-side arithmetic that kernels rely on, checked on the CPU: the multiply-high division
constants that the host precomputes for the index maps (`hck_fast_div_setup`, kargs.h) must give
exact quotients for every 32-bit numerator."""
import os
import shutil
import subprocess
import textwrap

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

PROGRAM = textwrap.dedent(r"""
    #include <stdint.h>
    #include <stdio.h>
    #include <stdlib.h>
    #include "kargs.h"
    /* the device side of the pair (common.hip.h: fast_div), restated with 64-bit host arithmetic */
    static uint32_t fast_div(uint32_t n, uint32_t magic, uint32_t sh) {
      const uint32_t t = (uint32_t)(((uint64_t)magic * n) >> 32);
      return (t + ((n - t) >> (sh & 0xffu))) >> (sh >> 8);
    }
    static uint64_t bad = 0, checks = 0;
    static void check(uint32_t n, uint32_t d) {
      uint32_t m, sh;
      hck_fast_div_setup(d, &m, &sh);
      checks++;
      if (fast_div(n, m, sh) != n / d) { if (bad++ < 10) printf("wrong: %u / %u\n", n, d); }
    }
    int main(void) {
      const uint32_t edge[] = {0, 1, 2, 3, 0x7fffffffu, 0x80000000u, 0x80000001u, 0xfffffffeu, 0xffffffffu};
      /* every divisor up to 4096 and around every power of two, against edge and nearby numerators */
      for (uint64_t d = 1; d <= 0xffffffffull; d = d < 4096 ? d + 1 : d + d / 3 + 1) {
        for (unsigned e = 0; e < sizeof(edge) / sizeof(edge[0]); e++) check(edge[e], (uint32_t)d);
        for (int64_t k = -2; k <= 2; k++)
          for (uint64_t mult = 1; mult <= 5; mult++) {
            const int64_t n = (int64_t)(d * mult) + k;
            if (n >= 0 && n <= 0xffffffffll) check((uint32_t)n, (uint32_t)d);
          }
      }
      for (int b = 1; b < 32; b++)
        for (int64_t k = -1; k <= 1; k++) {
          const uint32_t d = (uint32_t)((1ll << b) + k);
          for (unsigned e = 0; e < sizeof(edge) / sizeof(edge[0]); e++) check(edge[e], d);
        }
      srand(7);
      for (int i = 0; i < 2000000; i++) {
        uint32_t d = (((uint32_t)rand() << 16) ^ (uint32_t)rand()) >> (rand() % 32);
        const uint32_t n = ((uint32_t)rand() << 16) ^ (uint32_t)rand() ^ ((uint32_t)rand() << 31);
        check(n, d ? d : 1);
      }
      printf("%llu checks, %llu wrong\n", (unsigned long long)checks, (unsigned long long)bad);
      return bad != 0;
    }
""")


@pytest.mark.skipif(shutil.which("gcc") is None, reason="needs gcc")
def test_fast_division_constants_are_exact(tmp_path):
    src = tmp_path / "fastdiv.c"
    src.write_text(PROGRAM)
    exe = tmp_path / "fastdiv"
    subprocess.run(["gcc", "-O2", "-I", os.path.join(ROOT, "honeycrisp_amd", "csrc"), "-o", str(exe), str(src)],
                   check=True)
    out = subprocess.run([str(exe)], stdout=subprocess.PIPE, text=True)
    assert out.returncode == 0, out.stdout
    assert " 0 wrong" in out.stdout
