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
    tail = (B, H, Hk, Dh, S, nsplit, 0.0, stream)
    if static:
        return lib.fsvd_attn_decode_densekv_static(*head, *tail)
    return lib.fsvd_attn_decode_densekv(*head, ws.data_ptr(), ws.numel() * ws.element_size(), *tail)


def test_static_scratch_matches_workspace_entry_point_two_calls(lib):
    assert lib.fsvd_attn_decode_densekv_static_max_bytes() == 4 << 20
    # (B, H, Hk, Dh, S, keys, nsplit): the 7B decode shape first, then a smaller, ragged one on the same array
    cases = [(1, 32, 32, 128, 600, 513, 8), (2, 8, 4, 128, 96, 70, 4)]
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
        before = torch.cuda.memory_allocated()
        assert _call(lib, True, qg, kg, vg, lg, got_out, nsplit) == 0, lib.fsvd_last_error()
        assert torch.cuda.memory_allocated() == before
        torch.cuda.synchronize()
        assert torch.equal(got_out.view(torch.int16).cpu(), ref_out.view(torch.int16).cpu()), f"case {i}: bits differ"
        for b in range(B):
            k = int(lens[b])
            assert_close_bf16(got_out[b:b + 1], O.dense_decode_attn(q[b:b + 1], kc[b:b + 1, :k], vc[b:b + 1, :k]), f"case {i} b={b}")


def test_static_scratch_rejects_what_does_not_fit(lib):
    B, H, Dh, nsplit = 16, 32, 128, 64      # 16*32*64*130*4 B of partials: far beyond 4 MiB
    assert lib.fsvd_attn_decode_workspace_bytes(B, H, Dh, nsplit) > lib.fsvd_attn_decode_densekv_static_max_bytes()
    q = torch.zeros(B, H, Dh, dtype=torch.bfloat16, device="cuda")
    kc = torch.zeros(B, 64, H, Dh, dtype=torch.bfloat16, device="cuda")
    lens = torch.ones(B, dtype=torch.int32, device="cuda")
    rc = _call(lib, True, q, kc, kc, lens, torch.empty_like(q), nsplit)
    assert rc == -6 and b"scratch" in lib.fsvd_last_error()
