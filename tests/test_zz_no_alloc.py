"""mi_moe_forward_static: the forward that allocates nothing, on the library's built-in scratch.
Through the C ABI; its results must be mi_moe_forward's bit for bit, on two calls in a row (the
second on a smaller batch: the scratch still holds the first call's contents), and batches that need
more workspace than the scratch holds are refused with a message."""
import ctypes as C

import numpy as np
import pytest
import torch

from helpers import bf16_tensor, bits_u16, device_block, host_layer, host_tokens

pytestmark = pytest.mark.gpu


def _static(lib, m, blk, x):
    out = torch.empty_like(x)
    before = torch.cuda.memory_allocated()
    st = torch.cuda.current_stream().cuda_stream
    m.capi.check(lib.mi_moe_forward_static(blk._handle, x.data_ptr(), x.shape[0], out.data_ptr(), None, st))
    assert torch.cuda.memory_allocated() == before  # (torch's allocator; the library never calls it)
    return out


@pytest.mark.parametrize("H,E,k,I,bits,mode,batches", [
    (2048, 128, 8, 768, 4, 0, (32, 5)),    # the headline layer at decode: one-launch router, streamed experts
    (256, 8, 2, 512, 8, 2, (150, 40, 1)),  # tile lists and side streams, then light, then a single token
])
def test_static_scratch_forward_equals_forward(orc, H, E, k, I, bits, mode, batches):
    import mlx_rs_amd as m
    lib = m.load_library()
    W = host_layer(orc, H, E, k, I, bits, seed=123)
    blk = device_block(m, m.MoeConfig(H, E, k, I, bits, 64, mode), W)
    for T in batches:
        print(f"forward_static H={H} E={E} bits={bits} T={T}", flush=True)
        x = bf16_tensor(host_tokens(orc, T, H, seed=T), "cuda")
        want = blk.forward(x).clone()
        got = _static(lib, m, blk, x)
        torch.cuda.synchronize()
        assert np.array_equal(bits_u16(got), bits_u16(want)), f"T={T}: differs from mi_moe_forward"
    # the oracle agrees with the last batch too (not only the two entry points with each other)
    ref, _ = orc.moe_forward(orc.make_config(H, E, k, I, bits, 64, mode), W, host_tokens(orc, batches[-1], H, seed=batches[-1]),
                             strict=True, n_threads=8)
    from helpers import assert_close_bf16
    assert_close_bf16(bits_u16(got), ref, what="forward_static vs oracle")


def test_static_scratch_refuses_what_does_not_fit(orc):
    import mlx_rs_amd as m
    lib = m.load_library()
    H, E, k, I = 2048, 128, 8, 768
    W = host_layer(orc, H, E, k, I, 4, seed=5)
    blk = device_block(m, m.MoeConfig(H, E, k, I), W)
    T = 157  # one token more than 8 MiB of workspace serve for this layer (without the optional byte planes of the
             # int8 router logits, which mi_moe_workspace_size counts in: on the built-in scratch the logits of a batch
             # of more than 64 tokens come from the fp64 kernels, with the same bits)
    assert blk.workspace_bytes(T) - 256 > m.capi.STATIC_SCRATCH_BYTES
    x = bf16_tensor(host_tokens(orc, T, H, seed=1), "cuda")
    out = torch.full_like(x, 7.0)
    st = torch.cuda.current_stream().cuda_stream
    rc = lib.mi_moe_forward_static(blk._handle, x.data_ptr(), T, out.data_ptr(), None, st)
    assert rc != 0 and "built-in scratch" in m.capi.last_error()
    torch.cuda.synchronize()
    assert (out == 7.0).all(), "outputs touched by a refused call"
    got = blk.forward_static(x[:156].contiguous())  # the largest batch that fits
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), blk.forward(x[:156].contiguous()).view(torch.int16))
    with pytest.raises(m.MoeError, match="negative"):
        m.capi.check(lib.mi_moe_forward_static(blk._handle, x.data_ptr(), -1, out.data_ptr(), None, st))
