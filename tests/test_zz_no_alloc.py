"""The entry point that allocates nothing: ``iron_mha_decode_static_bf16`` against
``iron_mha_decode_bf16`` through the C ABI, bit for bit, two calls in a row on the library's one
scratch array, the second smaller than the first."""

import numpy as np
import pytest
import torch

from iron_amd import kernels as K
from iron_amd._lib import IronHipError, lib

pytestmark = pytest.mark.gpu


def test_decode_attention_from_the_library_s_own_scratch_is_the_workspace_one_bit_for_bit(cuda):
    g = torch.Generator(device=cuda)
    g.manual_seed(5)

    def bf(*shape):
        return torch.randn(shape, generator=g, device=cuda, dtype=torch.float32).to(torch.bfloat16)

    # The split kernel and its merge (over 2048 keys), then smaller calls on the same scratch: fewer
    # keys under a bound, fewer and wider heads, and the one-launch kernel (which leaves it untouched).
    cases = [(32, 8, 64, 16384, None, None), (32, 8, 64, 4096, 2500, None), (8, 2, 128, 2304, None, 700),
             (32, 8, 64, 1024, 900, None), (32, 8, 64, 16384, 16001, None)]
    warmed = False
    for H, G, d, L, bound, window in cases:
        Q, Kc, Vc = bf(1, H, d), bf(L, G, d), bf(L, G, d)
        kv_valid = None if bound is None else torch.tensor([bound], dtype=torch.int32, device=cuda)
        own = torch.full((1, H, d), float("nan"), dtype=torch.bfloat16, device=cuda)
        torch.cuda.synchronize()
        free, held = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
        K.mha_decode_static(Q, Kc, Vc, own, heads=H, kv_heads=G, d=d, kv_len=L, window=window, kv_interleaved=True,
                            kv_valid=kv_valid)
        torch.cuda.synchronize()
        if warmed:   # the first launch of a process may load the code object; no later one takes memory
            assert torch.cuda.mem_get_info()[0] == free and torch.cuda.memory_allocated() == held
        warmed = True
        ws = K.mha_decode_workspace(H, d, cuda)
        want = torch.full((1, H, d), float("nan"), dtype=torch.bfloat16, device=cuda)
        K.mha_decode(Q, Kc, Vc, want, heads=H, kv_heads=G, d=d, kv_len=L, window=window, kv_interleaved=True,
                     kv_valid=kv_valid, workspace=ws)
        torch.cuda.synchronize()
        assert not torch.isnan(own.float()).any()
        assert torch.equal(own, want), (H, G, d, L, bound, window)
    # Past the scratch's fixed size the call is refused with the reason, before any launch.
    limit = lib().iron_mha_decode_static_max_bytes()
    H, d = 256, 256
    assert lib().iron_mha_decode_workspace_bytes(H, d) > limit
    Q, Kc, Vc = bf(1, H, d), bf(64, H, d), bf(64, H, d)
    with pytest.raises(IronHipError, match="scratch holds"):
        K.mha_decode_static(Q, Kc, Vc, torch.empty_like(Q), heads=H, kv_heads=H, d=d, kv_len=64, kv_interleaved=True)


def test_static_decode_attention_under_graph_capture_after_one_warm_call(cuda):
    """What the entry point is for: once a call outside any capture has made the library look its
    scratch array's address up on this device, the call records into a HIP graph (it allocates
    nothing and asks the runtime nothing), and every replay is the workspace form bit for bit --
    replayed several times with eager work and synchronizations in between, new keys each time."""
    g = torch.Generator(device=cuda)
    g.manual_seed(6)

    def bf(*shape):
        return torch.randn(shape, generator=g, device=cuda, dtype=torch.float32).to(torch.bfloat16)

    H, G, d, L = 32, 8, 64, 6000
    Q, Kc, Vc = bf(1, H, d), bf(L, G, d), bf(L, G, d)
    kv_valid = torch.tensor([5000], dtype=torch.int32, device=cuda)
    own = torch.zeros((1, H, d), dtype=torch.bfloat16, device=cuda)

    def launch():
        K.mha_decode_static(Q, Kc, Vc, own, heads=H, kv_heads=G, d=d, kv_len=L, kv_interleaved=True, kv_valid=kv_valid)

    launch()   # the warm call
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            launch()
    torch.cuda.current_stream().wait_stream(stream)
    ws = K.mha_decode_workspace(H, d, cuda)
    for bound in (5000, 900, 6000, 2049):
        Kc.copy_(bf(L, G, d))
        kv_valid.fill_(bound)
        own.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        want = torch.empty_like(own)
        K.mha_decode(Q, Kc, Vc, want, heads=H, kv_heads=G, d=d, kv_len=L, kv_interleaved=True, kv_valid=kv_valid,
                     workspace=ws)
        torch.cuda.synchronize()
        assert torch.equal(own, want), bound
