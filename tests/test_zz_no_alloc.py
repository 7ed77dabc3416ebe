"""The entry point that allocates nothing (vui_decode_attn_noalloc) against vui_decode_attn, through the C ABI.

Same kernels, same inputs, the pieces merged in piece order: the outputs must be bit-identical.  Two calls in a
row share the library's built-in scratch array, the second with a smaller input, so whatever the first call left
there must not leak into the second."""
import gc

import pytest
import torch

from oracle import vui_oracle as O

pytestmark = pytest.mark.gpu

BF, F32 = torch.bfloat16, torch.float32


def _case(lib, dt, H, KV, hd, S, lens, splits, window, seed):
    from vui_amd import _lib

    st = torch.cuda.current_stream().cuda_stream
    B = len(lens)
    n_slots = B + 1
    g = torch.Generator().manual_seed(seed)
    slot_idx = torch.randperm(n_slots, generator=g)[:B].to(torch.int32)
    kc = torch.randn(n_slots, S, KV, hd, generator=g).to(dt).cuda()
    vc = torch.randn(n_slots, S, KV, hd, generator=g).to(dt).cuda()
    q = torch.randn(B, H, hd, generator=g).to(dt).cuda()
    kn = torch.randn(B, KV, hd, generator=g).to(dt).cuda()
    vn = torch.randn(B, KV, hd, generator=g).to(dt).cuda()
    seq_lens = torch.zeros(n_slots, dtype=torch.int32)
    for b, L in enumerate(lens):
        seq_lens[slot_idx[b]] = L
    sl, sid = seq_lens.cuda(), slot_idx.cuda()
    code = 1 if dt == F32 else 0
    # the existing entry point, with a scratch buffer of the caller
    kc1, vc1 = kc.clone(), vc.clone()
    want = torch.zeros(B, H, hd, dtype=dt, device="cuda")
    scratch = torch.zeros(lib.vui_attn_scratch_bytes(B, H, hd, splits), dtype=torch.uint8, device="cuda")
    _lib.check(lib.vui_decode_attn(code, q.data_ptr(), kn.data_ptr(), vn.data_ptr(), kc1.data_ptr(), vc1.data_ptr(),
                                   sl.data_ptr(), sid.data_ptr(), want.data_ptr(), B, H, KV, hd, S, window, splits,
                                   scratch.data_ptr(), st), "vui_decode_attn")
    # the new one
    kc2, vc2 = kc.clone(), vc.clone()
    got = torch.zeros(B, H, hd, dtype=dt, device="cuda")
    # "allocates nothing" is checked on the device's own count of free bytes, which a hipMalloc inside the library
    # would move (torch's counters only see torch's allocator); Python's collector is held off for the window so
    # that no tensor left behind by an earlier test is released inside it
    args = (code, q.data_ptr(), kn.data_ptr(), vn.data_ptr(), kc2.data_ptr(), vc2.data_ptr(), sl.data_ptr(),
            sid.data_ptr(), got.data_ptr(), B, H, KV, hd, S, window, splits, st)
    gc.collect()
    torch.cuda.synchronize()
    gc.disable()
    try:
        free_before = torch.cuda.mem_get_info()[0]
        reserved_before = torch.cuda.memory_reserved()
        rc = lib.vui_decode_attn_noalloc(*args)
        torch.cuda.synchronize()
        free_after = torch.cuda.mem_get_info()[0]
        reserved_after = torch.cuda.memory_reserved()
    finally:
        gc.enable()
    _lib.check(rc, "vui_decode_attn_noalloc")
    assert free_after >= free_before, (free_before, free_after)
    assert reserved_after == reserved_before
    assert torch.equal(got, want), float((got.float() - want.float()).abs().max())
    assert torch.equal(kc1, kc2) and torch.equal(vc1, vc2)  # the appended rows as well
    # and against the oracle, to the tolerance of the attention parity test
    ref = torch.zeros(B, H, hd)
    kcf, vcf = kc.float().cpu(), vc.float().cpu()
    for b, L in enumerate(lens):
        s = int(slot_idx[b])
        kk = torch.cat([kcf[s, :L], kn[b].float().cpu()[None]], 0).transpose(0, 1)
        vv = torch.cat([vcf[s, :L], vn[b].float().cpu()[None]], 0).transpose(0, 1)
        if window > 0:
            lo = max(0, L - window)
            kk, vv = kk[:, lo:], vv[:, lo:]
        kk, vv = kk.repeat_interleave(H // KV, 0), vv.repeat_interleave(H // KV, 0)
        ref[b] = O.attention(q[b].float().cpu()[:, None], kk, vv, hd ** -0.5, dt)[:, 0]
    tol = 2e-5 if dt == F32 else 2.0 ** -7
    assert (got.float().cpu() - ref).abs().max() <= tol * max(1.0, float(ref.abs().max()))


def _warm(lib):
    """One tiny call outside the measured windows: the first use of a kernel or of the built-in array in a process
    makes the HIP runtime load its code object, which takes device memory once and is not the entry point's doing."""
    st = torch.cuda.current_stream().cuda_stream
    z = torch.zeros(2, 1, 8, dtype=torch.float32, device="cuda")
    kc = torch.zeros(1, 4, 1, 8, dtype=torch.float32, device="cuda")
    vc = torch.zeros_like(kc)
    sl = torch.zeros(1, dtype=torch.int32, device="cuda")
    o = torch.zeros(1, 1, 8, dtype=torch.float32, device="cuda")
    for splits in (1, 2):
        rc = lib.vui_decode_attn_noalloc(1, z.data_ptr(), z.data_ptr(), z.data_ptr(), kc.data_ptr(), vc.data_ptr(),
                                         sl.data_ptr(), None, o.data_ptr(), 1, 1, 1, 8, 4, 0, splits, st)
        assert rc == 0
    torch.cuda.synchronize()


def test_noalloc_equals_decode_attn_two_calls_in_a_row():
    from vui_amd import _lib

    lib = _lib.load()
    _warm(lib)
    # first call: 16 ragged rows, 8 heads, 32 splits (the arrival counters and pieces of 128 (row, head) pairs)
    _case(lib, BF, 8, 8, 96, 2304, [2047, 128, 1500, 300, 777, 2100, 64, 1024, 999, 1, 0, 513, 1800, 256, 1337, 2200],
          32, 0, seed=1)
    # second call right after it, smaller in every respect, fp32: the array still holds the first call's pieces
    _case(lib, F32, 4, 2, 64, 200, [150, 3], 4, 0, seed=2)
    # one split (no pieces at all) and a sliding window
    _case(lib, BF, 8, 8, 96, 600, [500], 1, 0, seed=3)
    _case(lib, BF, 8, 4, 96, 600, [599, 17, 300], 8, 128, seed=4)


def test_noalloc_rejects_sizes_beyond_its_scratch():
    from vui_amd import _lib

    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    t = torch.zeros(64, dtype=torch.float32, device="cuda")
    p = t.data_ptr()
    # 16 rows x 16 heads x 64 splits x 130 floats = 8.5 MB of pieces: over the 4 MiB array
    rc = lib.vui_decode_attn_noalloc(0, p, None, None, p, p, p, None, p, 16, 16, 16, 128, 64, 0, 64, st)
    assert rc == -22 and "limit" in _lib.last_error()
    # more (row, head) pairs than counters
    rc = lib.vui_decode_attn_noalloc(0, p, None, None, p, p, p, None, p, 4096, 1, 1, 8, 64, 0, 1, st)
    assert rc == -22
