"""The C-ABI library loads on a machine without a GPU and exports every symbol include/picotron_amd.h declares.
Also the host-side logic that needs no GPU: schedule bookkeeping of the local ring and error behaviour."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "picotron_amd.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pico_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    syms = declared_symbols()
    for must in ("pico_attn_fwd", "pico_attn_bwd", "pico_attn_bwd_preprocess", "pico_lse_merge", "pico_rmsnorm_fwd",
                 "pico_rmsnorm_bwd", "pico_rope", "pico_swiglu_fwd", "pico_swiglu_bwd", "pico_version", "pico_last_error"):
        assert must in syms


def test_library_exports_every_declared_symbol():
    from picotron_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built here (python -m picotron_amd.build)")
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(handle, name), f"{name} declared in the header but not exported"
    assert set(_lib.SIGNATURES) == set(declared_symbols())
    lib = _lib.lib()
    assert lib.pico_version().decode().startswith("picotron_amd")


def test_argument_checks_run_without_a_gpu():
    """Validation happens before any launch, so bad arguments are reported even with no device."""
    from picotron_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built here")
    lib = _lib.lib()
    assert lib.pico_rmsnorm_fwd(None, None, None, None, None, None, 4, 7, 1e-5, 1, _lib.PICO_BF16, None) == -3
    assert b"hidden" in lib.pico_last_error()
    assert lib.pico_swiglu_fwd(None, None, None, 4, 8, 8, 8, 8, 99, None) == -2
    d = _lib.AttnDesc()
    d.B, d.Hq, d.Hkv, d.Sq, d.Sk, d.D, d.sm_scale = 1, 3, 2, 8, 8, 64, 0.125
    assert lib.pico_attn_fwd(ctypes.byref(d), None, None, None, None, None, 0, 0, None) == -3   # Hq % Hkv != 0
    d.Hkv, d.D = 3, 96
    assert lib.pico_attn_fwd(ctypes.byref(d), None, None, None, None, None, 0, 0, None) == -3   # head_dim
    assert b"head_dim" in lib.pico_last_error()
    assert lib.pico_rmsnorm_bwd_workspace_bytes(4096, 2048) == 512 * 2048 * 4
    # the kernels address one head's rows through 32-bit byte offsets: a 4 GiB span is refused
    d.D, d.Sq, d.Sk = 64, 64, 64
    for st in (d.q_stride, d.k_stride, d.v_stride, d.o_stride):
        st[0], st[1], st[2] = 64 * 64 * 3, 64 * 64, 64
    d.k_stride[2] = 1 << 26
    assert lib.pico_attn_fwd(ctypes.byref(d), None, None, None, None, None, 0, 0, None) == -5
    assert b"4 GiB" in lib.pico_last_error()


def test_argument_checks_of_the_optimizer_and_loss_entries():
    """Bad dtype codes, negative counts and sizes are refused before anything is launched (no device needed)."""
    from picotron_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built here")
    lib = _lib.lib()
    BF, F32 = _lib.PICO_BF16, _lib.PICO_F32
    hyper = (1e-3, 0.9, 0.999, 1e-8, 0.01)
    assert lib.pico_adamw(None, None, None, 99, None, None, 16, *hyper, 1, 1.0, None) == -2          # gradient dtype
    assert lib.pico_adamw(None, None, None, BF, None, None, 16, *hyper, 0, 1.0, None) == -3          # step counts from 1
    assert lib.pico_adamw(None, None, None, BF, None, None, 16, *hyper, 1, 1.0, None) == -1          # NULL state
    assert lib.pico_adamw(None, None, None, BF, None, None, 0, *hyper, 1, 1.0, None) == 0            # nothing to do
    assert lib.pico_adamw_lp(None, None, BF, None, None, 16, F32, F32, *hyper, 1, 1.0, None) == -2   # parameter must be bf16
    assert lib.pico_adamw_lp(None, None, BF, None, None, 16, BF, 7, *hyper, 1, 1.0, None) == -2      # state dtype
    assert lib.pico_adamw_multi(-1, None, None, None, None, None, None, BF, BF, BF, *hyper, 1, 1.0, None) == -3
    assert lib.pico_adamw_multi(0, None, None, None, None, None, None, BF, BF, BF, *hyper, 1, 1.0, None) == 0
    assert lib.pico_adamw_multi(2, None, None, None, None, None, None, BF, BF, BF, *hyper, 1, 1.0, None) == -1   # tables
    one = (ctypes.c_void_p * 1)(None)
    size = (ctypes.c_int64 * 1)(8)
    # fp32 weights with bf16 moments is not a layout the library has
    assert lib.pico_adamw_multi(1, one, None, one, one, one, size, F32, BF, BF, *hyper, 1, 1.0, None) == -2
    assert b"weight dtype" in lib.pico_last_error()
    size[0] = -4
    assert lib.pico_adamw_multi(1, one, None, one, one, one, size, BF, BF, BF, *hyper, 1, 1.0, None) == -3
    assert lib.pico_rmsnorm_bwd(None, None, None, None, None, None, None, 5, None, 0, 4, 64, BF, None) == -2     # dweight dtype
    assert lib.pico_cross_entropy_fwd(None, None, None, None, 4, 1000, 1003, -100, BF, None) != 0    # pitch not a multiple of 8


def test_cpu_tensors_are_refused_not_computed():
    from picotron_amd import ops
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.rmsnorm_fwd(torch.zeros(2, 8), torch.ones(8), 1e-5, True)
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.attn_fwd(*(torch.zeros(1, 1, 8, 64, dtype=torch.bfloat16) for _ in range(3)), 0.125, True)


def test_process_group_manager_stand_in():
    import picotron_amd.process_group_manager as pgm
    mgr = pgm.setup_process_group_manager(1, 4, 1, 1, cp_rank=2)
    assert (mgr.cp_rank, mgr.cp_world_size, mgr.cp_send_rank, mgr.cp_recv_rank) == (2, 4, 3, 1)
    assert mgr.tp_world_size == mgr.pp_world_size == mgr.dp_world_size == 1
    mgr.set_cp_rank(0)
    assert (mgr.cp_send_rank, mgr.cp_recv_rank) == (1, 3)          # ring neighbours wrap around
    with pytest.raises(AssertionError):
        pgm.setup_process_group_manager(2, 1, 1, 1)                # only cp may exceed 1 on one GPU
    pgm.setup_process_group_manager(1, 1, 1, 1)


C_PROGRAM = r"""
#include <stdio.h>
#include <string.h>
#include "picotron_amd.h"
int main(void) {
  pico_attn_desc d;
  memset(&d, 0, sizeof d);
  d.B = 1; d.Hq = 2; d.Hkv = 2; d.Sq = 8; d.Sk = 8; d.D = 48;   /* head_dim 48 is not supported */
  d.sm_scale = 0.125f;
  int rc = pico_attn_fwd(&d, (void*)16, (void*)16, (void*)16, (void*)16, (float*)16, PICO_BF16, 0, NULL);
  printf("%s|%d|%s\n", pico_version(), rc, pico_last_error());
  return rc == PICO_ERR_SHAPE ? 0 : 1;
}
"""


def test_header_is_plain_c_and_a_c_program_links_against_the_library(tmp_path):
    """include/picotron_amd.h compiles as C99 with -pedantic, and a C program built with gcc calls the library through
    it (an argument check that returns before any launch, so no GPU is needed)."""
    import shutil
    import subprocess
    from picotron_amd import _lib
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    inc = os.path.join(ROOT, "include")
    unit = tmp_path / "unit.c"
    unit.write_text('#include "picotron_amd.h"\nint main(void) { return 0; }\n')
    subprocess.run([gcc, "-std=c99", "-pedantic", "-Wall", "-Werror", "-fsyntax-only", "-I", inc, str(unit)], check=True)
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built here (python -m picotron_amd.build)")
    prog = tmp_path / "prog.c"
    prog.write_text(C_PROGRAM)
    exe = tmp_path / "prog"
    libdir = os.path.dirname(_lib.LIB_PATH)
    subprocess.run([gcc, "-std=c99", "-Wall", "-Werror", "-I", inc, str(prog), "-o", str(exe), "-L", libdir, "-lpicotron_amd",
                    "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib"], check=True)
    res = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stdout + res.stderr
    version, rc, message = res.stdout.strip().split("|", 2)
    assert version.startswith("picotron_amd") and int(rc) == -3 and "head_dim" in message
