"""GPU: the two measurement kernels of the bench-only probe library launch and reject bad requests
(they compute nothing that could be compared with an oracle; bench.py times them)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_probes_launch_and_check_arguments(dev):
    import bench
    from dlcompiler_amd import _lib

    lib = bench.load_probe_lib()
    stream = _lib.current_stream_ptr(dev)
    sink = torch.zeros(512, dtype=torch.float32, device=dev)
    sb = sink.numel() * 4
    blocks = 4
    nbytes = lib.dlb_probe_mfma_operand_bytes(blocks)
    assert nbytes == blocks * 512 * 256
    buf = torch.randn(nbytes // 2, device=dev).bfloat16()
    for fp8 in (0, 1):
        for valu in (0, 4, 8, 16):
            assert lib.dlb_probe_mfma_rate(buf.data_ptr(), nbytes, sink.data_ptr(), sb, blocks, fp8, 10, valu,
                                           stream) == 0
    assert lib.dlb_probe_mfma_rate(buf.data_ptr(), nbytes, sink.data_ptr(), sb, blocks, 0, 10, 5, stream) == -2
    assert lib.dlb_probe_mfma_rate(buf.data_ptr(), nbytes - 16, sink.data_ptr(), sb, blocks, 0, 10, 0, stream) == -4
    assert lib.dlb_probe_mfma_rate(buf.data_ptr(), nbytes, sink.data_ptr(), sb - 4, blocks, 0, 10, 0, stream) == -4
    assert lib.dlb_probe_mfma_rate(None, nbytes, sink.data_ptr(), sb, blocks, 0, 10, 0, stream) == -1
    assert lib.dlb_probe_hbm_read(buf.data_ptr(), sink.data_ptr(), sb, nbytes, stream) == 0
    assert lib.dlb_probe_hbm_read(buf.data_ptr(), sink.data_ptr(), sb, 24, stream) == -2
    assert lib.dlb_probe_hbm_read(buf.data_ptr(), sink.data_ptr(), 64, nbytes, stream) == -4
    torch.cuda.synchronize()
    assert (sink == 0).all()          # the sinks exist to keep the loops alive, not to be written
