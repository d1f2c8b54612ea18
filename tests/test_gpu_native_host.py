"""The C ABI from a host program that has no Python and no torch in it (tests/native/abi_host.cpp, built by
__graft_entry__.build()): it allocates with the HIP runtime, calls odit_rel_l1, odit_gated_residual, odit_adaln_modulate,
odit_qknorm_rope, odit_attn_fwd and odit_linear_rows through include/omni_dit.h and checks them against double-precision loops of its own."""

import subprocess
from pathlib import Path

import pytest

HOST = Path(__file__).resolve().parent / "native" / "abi_host.bin"


@pytest.mark.gpu
def test_native_host_program_through_the_c_abi(gpu):
    if not HOST.exists():  # normally built beforehand by __graft_entry__.build(); a host-only compile of seconds
        import __graft_entry__

        __graft_entry__.build_native_host_test()
    print(f"running {HOST}", flush=True)
    proc = subprocess.run([str(HOST)], capture_output=True, text=True, timeout=120)
    print(proc.stdout, proc.stderr, flush=True)
    assert proc.returncode == 0, f"exit status {proc.returncode}\n{proc.stdout}\n{proc.stderr}"
    for name in ("odit_rel_l1: ok", "odit_gated_residual: ok", "odit_adaln_modulate: ok", "odit_qknorm_rope: ok",
                 "odit_attn_fwd: ok", "odit_linear_rows: ok"):
        assert name in proc.stdout
