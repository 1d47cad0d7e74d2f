"""dlb_moe_align_block_size_static (the entry point that allocates nothing) against
dlb_moe_align_block_size, through the C ABI: bit-exact on two calls in a row, the second with a
smaller input, so anything the first call left in the library's static scratch would show."""
import pytest
import torch

from dlcompiler_amd import _lib

pytestmark = pytest.mark.gpu


def _buffers(numel, E, block, dev):
    cap = numel + E * (block - 1)
    nblk = max(1, -(-cap // block))
    mk = lambda n: torch.full((n,), -7, dtype=torch.int32, device=dev)
    return cap, nblk, mk(cap), mk(nblk), mk(E), mk(1)


def _align_pair(ids, E, block):
    """(outputs of the workspace entry point, outputs of the static-scratch entry point)."""
    lib = _lib.load()
    dev = ids.device
    numel = ids.numel()
    stream = _lib.current_stream_ptr(dev)
    cap, nblk, s0, e0, c0, n0 = _buffers(numel, E, block, dev)
    ws_bytes = lib.dlb_moe_align_ws_bytes(numel, E)
    ws = torch.empty((max(ws_bytes, 4) // 4,), dtype=torch.int32, device=dev)
    st = lib.dlb_moe_align_block_size(ids.data_ptr(), 0, numel, E, block, s0.data_ptr(), cap,
                                      e0.data_ptr(), nblk, c0.data_ptr(), n0.data_ptr(),
                                      ws.data_ptr(), ws.numel() * 4, stream)
    assert st == 0
    _, _, s1, e1, c1, n1 = _buffers(numel, E, block, dev)

    def call_static():
        st = lib.dlb_moe_align_block_size_static(ids.data_ptr(), 0, numel, E, block, s1.data_ptr(), cap,
                                                 e1.data_ptr(), nblk, c1.data_ptr(), n1.data_ptr(),
                                                 stream)
        assert st == 0
        torch.cuda.synchronize()

    # first call on this device: the module's code object and the address of the static array are
    # looked up here, once; the call after it must leave the device's free memory as it found it
    # (hipMemGetInfo sees every allocation, not only those of torch's caching allocator)
    call_static()
    before = torch.cuda.memory_allocated(dev)
    free_before = torch.cuda.mem_get_info(dev)[0]
    call_static()
    assert torch.cuda.memory_allocated(dev) == before
    assert torch.cuda.mem_get_info(dev)[0] == free_before
    return (s0, e0, c0, n0), (s1, e1, c1, n1)


def test_static_scratch_matches_workspace_entry_point(dev):
    from oracle import moe_gating as og

    g = torch.Generator().manual_seed(11)
    # two calls in a row on the same GPU: 16384 x 6 slots over 64 experts (48 chunks), then a
    # smaller one (700 x 2 slots over 8 experts: one chunk, stale rows left in the scratch)
    for T, K, E, block in ((16384, 6, 64, 64), (700, 2, 8, 16)):
        ids_cpu = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(torch.int32)
        ids = ids_cpu.to(dev).reshape(-1)
        ref, got = _align_pair(ids, E, block)
        for a, b in zip(ref, got):
            assert torch.equal(a, b)
        # and both agree with the CPU oracle
        rs, re_, rn, rc = og.align_block_size(ids_cpu, block, E)
        npad = int(rn.item())
        assert got[3].item() == npad
        assert torch.equal(got[0].cpu()[:npad], rs[:npad])
        assert torch.equal(got[1].cpu()[:npad // block], re_[:npad // block])
        assert torch.equal(got[2].cpu(), rc.to(torch.int32))


def test_static_scratch_rejects_oversized_input(dev):
    lib = _lib.load()
    limit = lib.dlb_moe_align_block_size_static_max_numel()
    assert limit == 256 * 2048
    numel, E, block = limit + 1, 8, 16
    cap = numel + E * (block - 1)
    nblk = -(-cap // block)
    ids = torch.zeros((numel,), dtype=torch.int32, device=dev)
    s = torch.empty((cap,), dtype=torch.int32, device=dev)
    e = torch.empty((nblk,), dtype=torch.int32, device=dev)
    n = torch.empty((1,), dtype=torch.int32, device=dev)
    st = lib.dlb_moe_align_block_size_static(ids.data_ptr(), 0, numel, E, block, s.data_ptr(), cap,
                                             e.data_ptr(), nblk, None, n.data_ptr(),
                                             _lib.current_stream_ptr(dev))
    assert st == -4  # DLB_ERR_WORKSPACE
