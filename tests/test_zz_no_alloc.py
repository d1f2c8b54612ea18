"""The no-allocation entry point ``odit_rel_l1_static`` (scratch in a fixed device array of the library)
against ``odit_rel_l1`` (caller's workspace), through the C ABI: bit-identical sums on two calls in a row,
the second on a smaller input, then on more shapes, on a side stream, and with poisoned scratch counters."""

import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu


def _pair(B, n, seed, dtype, gpu):
    g = torch.Generator().manual_seed(seed)
    prev = torch.randn(B, n, generator=g).to(dtype)
    cur = (prev.float() * 1.05 + 0.02 * torch.randn(B, n, generator=g)).to(dtype)
    return cur.to(gpu), prev.to(gpu)


def _with_workspace(lib, cur, prev, flags, stream):
    B, n = cur.shape
    need = int(lib.odit_rel_l1_workspace_bytes(B, n))
    ws = torch.zeros(need, dtype=torch.uint8, device=cur.device)
    sums = torch.full((B, 2), -1.0, dtype=torch.float64, device=cur.device)
    code = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}[cur.dtype]
    rc = lib.odit_rel_l1(cur.data_ptr(), prev.data_ptr(), sums.data_ptr(), ws.data_ptr(), need, B, n, cur.stride(0),
                         prev.stride(0), code, flags, stream)
    assert rc == 0, lib.odit_last_error()
    return sums


def _static(lib, cur, prev, flags, stream):
    B, n = cur.shape
    sums = torch.full((B, 2), -1.0, dtype=torch.float64, device=cur.device)
    code = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}[cur.dtype]
    rc = lib.odit_rel_l1_static(cur.data_ptr(), prev.data_ptr(), sums.data_ptr(), B, n, cur.stride(0), prev.stride(0),
                                code, flags, stream)
    assert rc == 0, lib.odit_last_error()
    return sums


def test_rel_l1_static_equals_the_workspace_entry_point(gpu):
    from vllm_omni_amd import _lib

    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    # two calls in a row, the second on a smaller input (fewer rows AND fewer workgroups per row)
    big = _pair(2, 4096 * 3072, 1, torch.bfloat16, gpu)
    small = _pair(1, 64 * 3072 + 5, 2, torch.bfloat16, gpu)
    print("odit_rel_l1_static: B=2 n=12582912 then B=1 n=196613", flush=True)
    got_big = _static(lib, *big, 1, stream)
    got_small = _static(lib, *small, 1, stream)
    torch.cuda.synchronize()
    want_big, want_small = _with_workspace(lib, *big, 1, stream), _with_workspace(lib, *small, 1, stream)
    torch.cuda.synchronize()
    assert torch.equal(got_big, want_big), (got_big, want_big)
    assert torch.equal(got_small, want_small), (got_small, want_small)
    # the sums themselves are right (difference rounded to bf16, as the flag asks)
    cur, prev = small
    sd = (cur - prev).abs().double().sum(dim=1)
    sp = prev.abs().double().sum(dim=1)
    assert torch.allclose(got_small[:, 0], sd, rtol=5e-6) and torch.allclose(got_small[:, 1], sp, rtol=5e-6)
    # more shapes and dtypes back to back, growing and shrinking, the row limit included
    for B, n, dtype, flags in ((64, 3000, torch.float32, 0), (3, 8 * 1024 * 8 + 5, torch.float16, 1),
                               (1, 7, torch.bfloat16, 0), (2, 4096 * 3072, torch.bfloat16, 0), (5, 100000, torch.float32, 0)):
        print(f"odit_rel_l1_static: B={B} n={n} {dtype}", flush=True)
        pair = _pair(B, n, B + n % 89, dtype, gpu)
        got = _static(lib, *pair, flags, stream)
        torch.cuda.synchronize()
        assert torch.equal(got, _with_workspace(lib, *pair, flags, stream)), (B, n, dtype)
    # a side stream (ordered against the default stream by the synchronisations around it)
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        got = _static(lib, *small, 1, side.cuda_stream)
    side.synchronize()
    assert torch.equal(got, want_small)


def test_rel_l1_static_clears_what_an_earlier_call_left(gpu):
    """The built-in array holds whatever the last launch on it left. Filled with garbage through a plain host-to-
    device copy (ticket words with huge launch numbers, which no atomic maximum of a later launch would override),
    the next calls still match the workspace entry point: each clears its ticket words first."""
    import ctypes as C

    from vllm_omni_amd import _lib

    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    nbytes = C.c_size_t(0)
    lib.odit_rel_l1_static_scratch.restype = C.c_void_p
    lib.odit_rel_l1_static_scratch.argtypes = [C.POINTER(C.c_size_t)]
    ptr = lib.odit_rel_l1_static_scratch(C.byref(nbytes))
    assert ptr and nbytes.value == 2560, lib.odit_last_error()
    hip = C.CDLL("libamdhip64.so")
    hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
    hip.hipMemcpy.restype = C.c_int
    torch.cuda.synchronize()
    dirt = (C.c_uint8 * nbytes.value)(*([0xEE] * nbytes.value))
    assert hip.hipMemcpy(ptr, dirt, nbytes.value, 1) == 0   # hipMemcpyHostToDevice
    for B, n, dtype, flags in ((64, 3000, torch.float32, 0), (2, 4096 * 3072, torch.bfloat16, 1)):
        print(f"odit_rel_l1_static on a dirtied array: B={B} n={n}", flush=True)
        pair = _pair(B, n, 9 + B, dtype, gpu)
        got = _static(lib, *pair, flags, stream)
        torch.cuda.synchronize()
        assert torch.equal(got, _with_workspace(lib, *pair, flags, stream))


def test_rel_l1_static_limits_and_errors(gpu):
    from vllm_omni_amd import _lib

    lib = _lib.load()
    cur, prev = _pair(65, 64, 3, torch.bfloat16, gpu)
    sums = torch.zeros(65, 2, dtype=torch.float64, device=gpu)
    rc = lib.odit_rel_l1_static(cur.data_ptr(), prev.data_ptr(), sums.data_ptr(), 65, 64, 64, 64, 0, 0, None)
    assert rc == -4 and b"64 rows" in lib.odit_last_error()
    rc = lib.odit_rel_l1_static(None, prev.data_ptr(), sums.data_ptr(), 1, 64, 64, 64, 0, 0, None)
    assert rc == -1
    rc = lib.odit_rel_l1_static(cur.data_ptr(), prev.data_ptr(), sums.data_ptr(), 1, 64, 64, 64, 7, 0, None)
    assert rc == -1 and b"dtype" in lib.odit_last_error()
    torch.cuda.synchronize()
