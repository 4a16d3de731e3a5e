"""The routing entry point that allocates nothing (moe355_init_routing_static) against the one that takes a
workspace (moe355_init_routing), through the C ABI: identical outputs on two calls in a row, the second with a
smaller batch (the fixed device array keeps the first call's contents)."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _route(lib, static, x, ids, E, quant_mode, tokens_num_type):
    from vllm_ascend_amd import _lib
    from vllm_ascend_amd.kernels import _stream

    T, k = ids.shape
    H = x.shape[1]
    R = T * k
    dev = x.device
    # outputs pre-filled, so that an entry a call fails to write shows up as a difference
    xs = torch.full((R, H), 77, dtype=torch.int8 if quant_mode == 1 else x.dtype, device=dev)
    row_idx = torch.full((R,), -5, dtype=torch.int32, device=dev)
    tokens = torch.full((E,), -5, dtype=torch.int64, device=dev)
    scale = torch.full((R,), -5.0, dtype=torch.float32, device=dev)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    if static:
        rc = lib.moe355_init_routing_static(p(x), _lib.DT_BF16, T, H, p(ids), k, E, quant_mode, tokens_num_type, p(xs),
                                            p(row_idx), p(tokens), p(scale), _stream(x))
    else:
        n = lib.moe355_init_routing_workspace(T, k, E)
        ws = torch.empty(n, dtype=torch.uint8, device=dev)
        rc = lib.moe355_init_routing(p(x), _lib.DT_BF16, T, H, p(ids), k, E, quant_mode, tokens_num_type, p(xs),
                                     p(row_idx), p(tokens), p(scale), p(ws), n, _stream(x))
    assert rc == 0, lib.moe355_strerror(rc)
    torch.cuda.synchronize()
    return xs, row_idx, tokens, scale


def test_static_routing_matches_the_workspace_form_on_two_calls_in_a_row():
    from vllm_ascend_amd import _lib

    lib = _lib.load()
    dev = "cuda:0"
    g = torch.Generator().manual_seed(11)
    # (tokens, top_k, experts, hidden, quant_mode, tokens_num_type): a batch that takes the histogram / scan /
    # scatter kernels, then a smaller one of the same kind, then one small enough for the single-launch form
    for T, k, E, H, qm, tt in [(1500, 8, 128, 512, 1, 1), (700, 8, 128, 512, 1, 0), (40, 4, 64, 256, -1, 1)]:
        x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
        ids = torch.randint(0, E, (T, k), generator=g, dtype=torch.int32).to(dev)
        want = _route(lib, False, x, ids, E, qm, tt)
        got = _route(lib, True, x, ids, E, qm, tt)
        for name, a, b in zip(("expanded_x", "expanded_row_idx", "expert_tokens", "dynamic_scale"), got, want):
            if name == "dynamic_scale" and qm != 1:
                continue
            assert torch.equal(a.view(torch.uint8) if a.dtype == torch.bfloat16 else a,
                               b.view(torch.uint8) if b.dtype == torch.bfloat16 else b), (name, T, k, E)


def test_static_routing_rejects_batches_beyond_its_array():
    from vllm_ascend_amd import _lib

    lib = _lib.load()
    one = ctypes.c_void_p(256)  # never dereferenced: the call is refused on the host
    T, k, E = 1 << 20, 8, 2048
    assert lib.moe355_init_routing_workspace(T, k, E) > (2 << 20)
    assert lib.moe355_init_routing_static(one, _lib.DT_BF16, T, 64, one, k, E, 1, 1, one, one, one, one, None) == -3
