"""The attention backward entry point that allocates nothing (tgk_attn_bwd_static: its two row vectors live in
a device array inside the library) against tgk_attn_bwd with a caller's workspace, through the C ABI.  Both
run the same deterministic kernels, so the bar is bit equality; two calls in a row share the array, the second
with a smaller input."""
import numpy as np
import pytest
import torch

from gpu_util import check, library, stream, sync, to_bf16_device

pytestmark = pytest.mark.gpu


def backward_pair(B, H, T, seed):
    lib = library()
    d = H * 64
    rng = np.random.default_rng(seed)
    qkv, _ = to_bf16_device(rng.standard_normal((B * T, 3 * d)))
    do, _ = to_bf16_device(rng.standard_normal((B * T, d)))
    o = torch.empty(B * T, d, dtype=torch.bfloat16, device="cuda")
    lse = torch.empty(B, H, T, dtype=torch.float32, device="cuda")
    p = qkv.data_ptr()
    check(lib.tgk_attn_fwd(stream(), B, H, T, 64, p, p + 2 * d, p + 4 * d, 3 * d, o.data_ptr(), d, lse.data_ptr(),
                           0.125))
    need = lib.tgk_attn_bwd_workspace(B, H, T)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    want = torch.zeros(B * T, 3 * d, dtype=torch.bfloat16, device="cuda")
    got = torch.zeros_like(want)
    g = want.data_ptr()
    check(lib.tgk_attn_bwd(stream(), B, H, T, 64, p, p + 2 * d, p + 4 * d, 3 * d, o.data_ptr(), d, lse.data_ptr(),
                           do.data_ptr(), d, g, g + 2 * d, g + 4 * d, 3 * d, 0.125, ws.data_ptr(), need))
    g = got.data_ptr()
    check(lib.tgk_attn_bwd_static(stream(), B, H, T, 64, p, p + 2 * d, p + 4 * d, 3 * d, o.data_ptr(), d,
                                  lse.data_ptr(), do.data_ptr(), d, g, g + 2 * d, g + 4 * d, 3 * d, 0.125))
    sync()
    return got, want


def test_static_scratch_backward_equals_the_workspace_backward_twice_in_a_row():
    for B, H, T, seed in [(2, 3, 512, 5), (1, 2, 128, 6)]:  # the second call is smaller and reuses the array
        print(f"attn_bwd_static B={B} H={H} T={T} seed={seed}", flush=True)
        got, want = backward_pair(B, H, T, seed)
        assert float(want.float().abs().sum()) > 0
        assert torch.equal(got, want)


def test_static_scratch_backward_rejects_what_does_not_fit():
    lib = library()
    rows = lib.tgk_attn_bwd_static_max_rows()
    assert rows == 1 << 20
    one = torch.zeros(16, dtype=torch.bfloat16, device="cuda").data_ptr()
    # 2 * 8 * 65664 rows > 2^20: rejected on the host, nothing is launched
    assert lib.tgk_attn_bwd_static(stream(), 2, 8, 65664, 64, one, one, one, 8, one, 8, one, one, 8, one, one, one,
                                   8, 0.125) == -1
    assert b"exceeds" in lib.tgk_error()
