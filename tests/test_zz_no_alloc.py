"""The allocation-free attention entry point (fsvd_attn_decode_densekv_static: scratch in a fixed array that the
library owns) against fsvd_attn_decode_densekv with a caller-owned workspace, both through the C ABI.

Same kernels, same split order: the outputs must be bit-identical, and both must meet the decode tolerance against
the CPU oracle.  Two calls in a row share the array, the second on a smaller input."""
import ctypes

import pytest
import torch

from oracle import flashsvd_oracle as O
from tests.util import assert_close_bf16, rand_bf16

pytestmark = pytest.mark.gpu


def _call(lib, static, q, kc, vc, lens, out, nsplit, ws=None):
    B, H, Dh = q.shape
    S, Hk = kc.shape[1], kc.shape[2]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    head = (q.data_ptr(), q.stride(0), q.stride(1), kc.data_ptr(), vc.data_ptr(), kc.stride(0), kc.stride(1), kc.stride(2),
            None, 0, 0, None, 0, 0, lens.data_ptr(), 0, None, None, 0, out.data_ptr(), out.stride(0), out.stride(1))
    tail = (B, H, Hk, Dh, S, nsplit, 0.0, 0, stream)
    if static:
        return lib.fsvd_attn_decode_densekv_static(*head, *tail)
    return lib.fsvd_attn_decode_densekv(*head, ws.data_ptr(), ws.numel() * ws.element_size(), *tail)


def test_static_scratch_matches_workspace_entry_point_two_calls(lib):
    assert lib.fsvd_attn_decode_densekv_static_max_bytes() == 4 << 20
    # (B, H, Hk, Dh, S, keys, nsplit): the 7B decode shape first, then a smaller, ragged one on the same array, then a
    # grouped-query batch large enough for the kernel that takes four query heads of a kv head per workgroup, and a call
    # without key splits (no scratch at all)
    cases = [(1, 32, 32, 128, 600, 513, 8), (2, 8, 4, 128, 96, 70, 4), (16, 32, 8, 128, 300, 257, 4), (2, 8, 4, 128, 96, 70, 1)]
    for i, (B, H, Hk, Dh, S, n, nsplit) in enumerate(cases):
        q = rand_bf16(B, H, Dh, seed=10 + i)
        kc, vc = rand_bf16(B, S, Hk, Dh, seed=20 + i), rand_bf16(B, S, Hk, Dh, seed=30 + i)
        lens = torch.tensor([max(1, n - 9 * b) for b in range(B)], dtype=torch.int32)
        qg, kg, vg, lg = q.cuda(), kc.cuda(), vc.cuda(), lens.cuda()
        need = lib.fsvd_attn_decode_workspace_bytes(B, H, Dh, nsplit)
        ws = torch.zeros(need // 4, dtype=torch.int32, device="cuda")
        ref_out = torch.empty(B, H, Dh, dtype=torch.bfloat16, device="cuda")
        got_out = torch.full((B, H, Dh), float("nan"), dtype=torch.bfloat16, device="cuda")
        assert _call(lib, False, qg, kg, vg, lg, ref_out, nsplit, ws) == 0, lib.fsvd_last_error()
        torch.cuda.synchronize()
        before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
        assert _call(lib, True, qg, kg, vg, lg, got_out, nsplit) == 0, lib.fsvd_last_error()
        torch.cuda.synchronize()
        # torch's allocator and the driver agree that nothing was allocated: the second figure also sees a hipMalloc made
        # inside the library (the first static call of the process has run by now: the array's address is taken then)
        assert torch.cuda.memory_allocated() == before
        if i > 0:
            assert torch.cuda.mem_get_info()[0] == free_before
        assert torch.equal(got_out.view(torch.int16).cpu(), ref_out.view(torch.int16).cpu()), f"case {i}: bits differ"
        for b in range(B):
            k = int(lens[b])
            assert_close_bf16(got_out[b:b + 1], O.dense_decode_attn(q[b:b + 1], kc[b:b + 1, :k], vc[b:b + 1, :k]), f"case {i} b={b}")


def test_static_call_under_stream_capture(lib):
    """The entry point clears its counters with a fill kernel, not a memset node, so that a caller under HIP stream
    capture can record it: two replays on changed cache lengths, each checked against the eager workspace call."""
    B, H, Hk, Dh, S, nsplit = 2, 16, 4, 128, 200, 4
    q = rand_bf16(B, H, Dh, seed=41).cuda()
    kc, vc = rand_bf16(B, S, Hk, Dh, seed=42).cuda(), rand_bf16(B, S, Hk, Dh, seed=43).cuda()
    lens = torch.tensor([150, 33], dtype=torch.int32, device="cuda")
    out = torch.empty(B, H, Dh, dtype=torch.bfloat16, device="cuda")
    ref = torch.empty_like(out)
    ws = torch.zeros(lib.fsvd_attn_decode_workspace_bytes(B, H, Dh, nsplit) // 4, dtype=torch.int32, device="cuda")
    assert _call(lib, True, q, kc, vc, lens, out, nsplit) == 0, lib.fsvd_last_error()      # warm-up outside the capture
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        assert _call(lib, True, q, kc, vc, lens, out, nsplit) == 0, lib.fsvd_last_error()
    for new_lens in ([150, 33], [199, 1], [64, 128]):
        lens.copy_(torch.tensor(new_lens, dtype=torch.int32))
        out.fill_(float("nan"))
        g.replay()
        assert _call(lib, False, q, kc, vc, lens, ref, nsplit, ws) == 0, lib.fsvd_last_error()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16)), f"replay with lengths {new_lens}: bits differ"


def test_static_scratch_rejects_what_does_not_fit(lib):
    B, H, Dh, nsplit = 16, 32, 128, 64      # 16*32*64*130*4 B of partials: far beyond 4 MiB
    assert lib.fsvd_attn_decode_workspace_bytes(B, H, Dh, nsplit) > lib.fsvd_attn_decode_densekv_static_max_bytes()
    q = torch.zeros(B, H, Dh, dtype=torch.bfloat16, device="cuda")
    kc = torch.zeros(B, 64, H, Dh, dtype=torch.bfloat16, device="cuda")
    lens = torch.ones(B, dtype=torch.int32, device="cuda")
    rc = _call(lib, True, q, kc, kc, lens, torch.empty_like(q), nsplit)
    assert rc == -6 and b"scratch" in lib.fsvd_last_error()
