"""The allocation-free decode-attention entry (nc_decode_attention_static) through the C ABI: same results, bit for bit, as
nc_decode_attention with a caller's workspace, on two calls in a row (the second smaller, so that it meets what the first
left in the built-in scratch), and a refusal beyond the stated maximum."""
import ctypes as C
import sys

import pytest
import torch

from nanochat_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda"


def say(msg):
    print(f"[gpu-case] {msg}", flush=True)
    sys.stdout.flush()


def ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def both_entries(B, T, H, Hkv, Tmax, window, splits, seed):
    lib = _lib.lib()
    g = torch.Generator(device=DEV).manual_seed(seed)
    kc = torch.randn(B, Tmax, Hkv, 128, generator=g, device=DEV).bfloat16()
    vc = torch.randn(B, Tmax, Hkv, 128, generator=g, device=DEV).bfloat16()
    q = (torch.randn(B, T, H, 128, generator=g, device=DEV) * 1.5).bfloat16()
    seq = torch.randint(0, Tmax - T + 1, (B,), generator=g, device=DEV).to(torch.int32)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    ws_bytes = lib.nc_attention_workspace_bytes(B, T, H, Tmax)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=DEV)
    want = torch.full_like(q, float("nan"))
    got = torch.full_like(q, float("nan"))
    amax_a = torch.zeros(1, dtype=torch.int32, device=DEV)
    amax_b = torch.zeros(1, dtype=torch.int32, device=DEV)
    _lib.check(lib.nc_decode_attention(ptr(q), ptr(kc), ptr(vc), ptr(seq), window, ptr(want), B, T, H, Hkv, Tmax, 0, ptr(ws), ws_bytes,
                                       ptr(amax_a), splits, stream))
    # everything the entry point needs exists by now: from here to the comparison nothing may be allocated
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    free_before = torch.cuda.mem_get_info()[0]           # what the driver reports: sees a hipMalloc that torch's allocator would not
    _lib.check(lib.nc_decode_attention_static(ptr(q), ptr(kc), ptr(vc), ptr(seq), window, ptr(got), B, T, H, Hkv, Tmax, 0, ptr(amax_b),
                                              splits, stream))
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
    torch.cuda.synchronize()
    # the scratch is 8.65 MB: had the call (or the runtime on its behalf) allocated it, the device's free memory would show it
    assert free_before - torch.cuda.mem_get_info()[0] < (1 << 20), (free_before, torch.cuda.mem_get_info()[0])
    assert torch.isfinite(want.float()).all()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (got.float() - want.float()).abs().max().item()
    assert amax_a.item() == amax_b.item() and amax_a.item() != 0


def test_static_scratch_entry_matches_the_workspace_entry_twice_in_a_row():
    say("nc_decode_attention_static: 6 rows x 13 heads, 8 splits, then a smaller call")
    lib = _lib.lib()
    assert lib.nc_decode_attention_static_max_row_heads() == 1024
    splits, _ = C.c_int(0), None
    heads = C.c_int(0)
    _lib.check(lib.nc_decode_attention_plan(6, 1, 13, -1, 700, 0, C.byref(splits), C.byref(heads)))
    assert splits.value > 1, "the first call was meant to split its keys over workgroups (the case that uses the scratch)"
    # one call ahead of the measured ones: the first use of the library's device code (its module, with the scratch array in it, is
    # loaded then) is not what the memory checks below are about
    warm = torch.zeros(1, 1, 2, 128, dtype=torch.bfloat16, device=DEV)
    wkv = torch.zeros(1, 8, 2, 128, dtype=torch.bfloat16, device=DEV)
    _lib.check(lib.nc_decode_attention_static(ptr(warm), ptr(wkv), ptr(wkv), ptr(torch.zeros(1, dtype=torch.int32, device=DEV)), -1,
                                              ptr(torch.empty_like(warm)), 1, 1, 2, 2, 8, 0, None, 0,
                                              C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    both_entries(6, 1, 13, 13, 700, -1, 0, seed=1)                # chosen split count (> 1): counters and partials in use
    both_entries(2, 1, 4, 2, 300, 64, 4, seed=2)                  # smaller, right behind it, on what the first call left
    both_entries(3, 3, 8, 2, 200, -1, 16, seed=3)                 # several queries per row, the maximum split count
    both_entries(64, 1, 16, 4, 128, -1, 0, seed=4)                # exactly the maximum: 64 * 16 = 1024 (row, head) pairs


def test_static_scratch_entry_refuses_what_does_not_fit():
    say("nc_decode_attention_static: refusal beyond the maximum")
    lib = _lib.lib()
    B, H, Tmax = 80, 13, 64                                        # 1040 (row, head) pairs
    q = torch.zeros(B, 1, H, 128, dtype=torch.bfloat16, device=DEV)
    kc = torch.zeros(B, Tmax, H, 128, dtype=torch.bfloat16, device=DEV)
    seq = torch.zeros(B, dtype=torch.int32, device=DEV)
    out = torch.empty_like(q)
    rc = lib.nc_decode_attention_static(ptr(q), ptr(kc), ptr(kc), ptr(seq), -1, ptr(out), B, 1, H, H, Tmax, 0, None, 0,
                                        C.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == -1 and b"exceed the built-in scratch" in lib.nc_last_error()
    torch.cuda.synchronize()
