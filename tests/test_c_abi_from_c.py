"""The boundary is a C ABI: include/ps_adam.h must compile as plain C (not only as C++), and a C program must be
able to link the library and drive its host-side entry points.  No GPU is needed: only calls that are answered on the
host (registry, argument checks) are made."""
import os
import shutil
import subprocess

import pytest

from patrickstar_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

C_SOURCE = r"""
#include <stdio.h>
#include <string.h>
#include "ps_adam.h"

int main(void)
{
    ps_chunk bad;
    ps_step_state st;
    int rc;
    if (sizeof(ps_chunk) != 32 || sizeof(ps_step_state) != 256 || sizeof(ps_call_pattern) != 32 || sizeof(ps_scale_record) != 16) return 10;
    if (ps_abi_version() != PS_ABI_VERSION) return 11;
    if (ps_adam_create(4242, 1e-3f, 0.9f, 0.999f, 1e-8f, 0.01f, 1, 0) != 0) return 12;
    if (ps_adam_set_arithmetic(4242, PS_ARITH_TORCH) != 0) return 13;
    if (ps_adam_set_arithmetic(4242, 5) != PS_ERR_BAD_ARG) return 14;
    memset(&bad, 0, sizeof bad);
    rc = ps_adam_step_chunks(4242, 1, 1e-3, 0.9, 0.999, 1e-8, 0.01, 1, &bad, 1, 1024, NULL, NULL, 4096.0, NULL);
    if (rc != PS_ERR_BAD_ARG || strstr(ps_last_error(), "NULL payload") == NULL) return 15;
    if (ps_adam_step_chunks(4243, 1, 1e-3, 0.9, 0.999, 1e-8, 0.01, 1, &bad, 0, 1024, NULL, NULL, 4096.0, NULL) != PS_ERR_UNKNOWN_ID) return 16;
    if (ps_state_read(NULL, &st, NULL) != PS_ERR_BAD_ARG) return 17;
    if (ps_adam_destroy(4242) != 0) return 18;
    puts("c abi ok");
    return 0;
}
"""


@pytest.mark.skipif(shutil.which("gcc") is None, reason="gcc not found")
def test_header_is_plain_c_and_a_c_program_links_the_library(tmp_path):
    src = tmp_path / "abi.c"
    src.write_text(C_SOURCE)
    include = os.path.join(ROOT, "include")
    # the header alone, strict ISO C
    subprocess.check_call(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-I", include,
                           "-x", "c", os.path.join(include, "ps_adam.h")])
    assert os.path.exists(_lib.LIB_PATH), "build the HIP library first (python -m patrickstar_amd.build)"
    exe = tmp_path / "abi"
    libdir = os.path.dirname(_lib.LIB_PATH)
    subprocess.check_call(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-I", include, str(src), "-o",
                           str(exe), "-L", libdir, "-lps_adam", "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib"])
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "c abi ok" in r.stdout, (r.returncode, r.stdout, r.stderr)
