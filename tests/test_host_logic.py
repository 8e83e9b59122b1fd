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


def test_code_objects_hold_every_reduce_and_gemm_kernel_the_host_names():
    """The host builds kernel names from (form, op, dtype) at run time and looks them up in the
    embedded code objects; a family that was dropped from a source file would only show on a GPU.
    The names are plain strings in the built code objects."""
    import itertools
    build = os.path.join(ROOT, "honeycrisp_amd", "csrc", "build")
    blob = {}
    for name in ("reduce", "gemm", "gemm_dma", "gemm_dma2", "gemm_mi16", "elementwise", "gather"):
        path = os.path.join(build, name + ".hsaco")
        if not os.path.exists(path):
            pytest.skip("code objects not built")
        blob[name] = open(path, "rb").read()
    forms = ["rows1", "rows8", "rows64", "rows256", "rowsplit", "cols"]
    for form, op, dt in itertools.product(forms, ["sum", "prod", "argmax", "argmin"], ["f32", "f16", "i64", "b8"]):
        names = ["hc_reduce_%s_%s_%s" % (form, op, dt)] if form != "cols" else \
            ["hc_reduce_cols_%s_%s_v1" % (op, dt), "hc_reduce_cols_%s_%s_vN" % (op, dt), "hc_reduce_cols_final_%s_%s" % (op, dt)]
        if op.startswith("arg") and form.startswith("rows") and form != "rowsplit":   # the form that also leaves the extremum itself
            names.append("hc_reduce_%s_%s_value_%s" % (form, op, dt))
        for n in names:
            assert n.encode() + b"\0" in blob["reduce"], n
    layouts = ["kk", "kn", "mk", "mn"]
    for tile, lay, edge in itertools.product(["256x256", "256x192", "192x256", "192x192", "256x128", "128x128", "256x64",
                                              "128x64", "64x64"], layouts, ["", "_e"]):
        assert ("hc_gemm_f16_mi16_%s_%s%s" % (tile, lay, edge)).encode() + b"\0" in blob["gemm_mi16"]
    for pipe, dt, tile, lay, edge in itertools.product(["dma", "dma2"], ["f16", "f32"],
                                                       ["256x256", "256x128", "128x128", "256x64", "128x64", "64x64"],
                                                       layouts, ["", "_e"]):
        assert ("hc_gemm_%s_%s_%s_%s%s" % (dt, pipe, tile, lay, edge)).encode() + b"\0" in blob["gemm_" + pipe]
    for dt in ("f16", "f32"):
        for n in ("hc_gemm_%s_xx", "hc_gemm_%s_kk", "hc_gemm_skinny_k_%s_q4", "hc_gemm_skinny_p_%s_q4",
                  "hc_gemm_skinny_pack_%s", "hc_gemm_skinny_store_%s", "hc_gemm_skinny_pair_%s", "hc_copy2d_pad_b%d", "hc_copy2d_unpad_b%d"):
            name = n % (dt if "%s" in n else (2 if dt == "f16" else 4))
            assert any(name.encode() + b"\0" in b for b in blob.values()), name


def test_build_refuses_register_tiled_kernels_that_use_scratch_memory():
    """The build reads the compiler's resource remarks for the tiled GEMM code objects: a kernel
    whose accumulators ended up in private memory still gives correct results, only several
    times slower, so no parity test would notice it."""
    from honeycrisp_amd.csrc import build
    remarks = textwrap.dedent("""\
        k.hip:9:1: remark: Function Name: hc_gemm_a [-Rpass-analysis=kernel-resource-usage]
        k.hip:9:1: remark:     VGPRs: 110 [-Rpass-analysis=kernel-resource-usage]
        k.hip:9:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]
        k.hip:9:1: remark: Function Name: hc_gemm_b [-Rpass-analysis=kernel-resource-usage]
        k.hip:9:1: remark:     ScratchSize [bytes/lane]: 1088 [-Rpass-analysis=kernel-resource-usage]
        k.hip:9:1: remark: Function Name: hc_gemm_c [-Rpass-analysis=kernel-resource-usage]
        k.hip:9:1: remark:     ScratchSize [bytes/lane]: 68 [-Rpass-analysis=kernel-resource-usage]
        """)
    assert build.kernels_with_scratch(remarks, 128) == ["hc_gemm_b (1088 bytes/lane)"]
    assert build.kernels_with_scratch(remarks, 16) == ["hc_gemm_b (1088 bytes/lane)", "hc_gemm_c (68 bytes/lane)"]
    lds = textwrap.dedent("""\
        k.hip:9:1: remark: Function Name: hc_gemm_a [-Rpass-analysis=kernel-resource-usage]
        k.hip:9:1: remark:     LDS Size [bytes/block]: 65536 [-Rpass-analysis=kernel-resource-usage]
        k.hip:9:1: remark: Function Name: hc_gemm_b [-Rpass-analysis=kernel-resource-usage]
        k.hip:9:1: remark:     LDS Size [bytes/block]: 71680 [-Rpass-analysis=kernel-resource-usage]
        """)
    assert build.kernels_with_promoted_private_data(lds) == ["hc_gemm_b (71680 bytes of LDS)"]
    assert {"gemm_dma", "gemm_dma2", "gemm_mi16", "gemm_mi16_m"} <= set(build.NO_SCRATCH)
    assert set(build.NO_SCRATCH) <= {name for name, _src, _flags in build.KERNELS}
