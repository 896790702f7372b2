"""The boundary as a C program sees it: ``include/pa_amd.h`` compiles as C99 and as C++17 without warnings, and a C
program linked against ``libpa_amd.so`` calls host-only entry points (no GPU needed) and gets the checker's answers."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INC = os.path.join(ROOT, "include")
LIB_DIR = os.path.join(ROOT, "openvino.genai_amd", "csrc")

C_PROGRAM = r"""
#include <stdio.h>
#include <string.h>
#include "pa_amd.h"

int main(void) {
    /* two sequences: a decode step behind 100 tokens of which 32 were evicted, and a 40-token chunk from scratch */
    const int64_t processed[2] = {100, 0}, evicted[2] = {32, 0}, skipped[2] = {0, 0}, scheduled[2] = {1, 40};
    const int64_t blocks[2] = {3, 2};
    int32_t past[2], sb[3], bib[3], max_ctx = -1;
    const int32_t rc = pa_pack_step(2, processed, evicted, skipped, scheduled, blocks, 32, past, sb, bib, &max_ctx);
    printf("%d %d %d %d %d %d %d %d %d %d\n", rc, past[0], past[1], sb[0], sb[1], sb[2], bib[0], bib[1], bib[2], max_ctx);
    /* SnapKV window 8, prompt 100: a chunk of 16 tokens behind 80 processed ones straddles the window's start */
    printf("%llu\n", (unsigned long long)pa_snapkv_num_scores(8, 100, 16, 80));
    /* a bad argument comes back as a status, never as an exception or a crash */
    printf("%d\n", pa_pack_step(2, processed, evicted, skipped, scheduled, blocks, 0, past, sb, bib, &max_ctx) != 0);
    printf("%s\n", strlen(pa_version()) > 0 ? "version" : "");
    return 0;
}
"""


@pytest.mark.parametrize("compiler,std", [("gcc", "-std=c99"), ("g++", "-std=c++17")])
def test_header_compiles_without_warnings(tmp_path, compiler, std):
    if shutil.which(compiler) is None:
        pytest.skip(f"{compiler} not installed")
    src = tmp_path / ("t.c" if compiler == "gcc" else "t.cpp")
    src.write_text('#include "pa_amd.h"\nint main(void) { return 0; }\n')
    r = subprocess.run([compiler, std, "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", f"-I{INC}", str(src)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


def test_c_program_links_and_calls_the_library(tmp_path, pkg):
    if shutil.which("gcc") is None:
        pytest.skip("gcc not installed")
    src = tmp_path / "use.c"
    src.write_text(C_PROGRAM)
    exe = tmp_path / "use"
    r = subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", f"-I{INC}", str(src), "-o", str(exe), f"-L{LIB_DIR}",
                        "-lpa_amd", f"-Wl,-rpath,{LIB_DIR}", "-Wl,-rpath,/opt/rocm/lib"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    lines = out.stdout.split("\n")
    # past = processed - evicted; prefix sums of scheduled tokens and of blocks; max context = processed + scheduled
    assert lines[0].split() == ["0", "68", "0", "0", "1", "41", "0", "3", "5", "101"], lines[0]
    assert lines[1] == "4"      # tokens 92 .. 95 of the chunk lie inside the last 8 of the prompt
    assert lines[2] == "1"
    assert lines[3] == "version"
