"""The two measurement aids of the C ABI (msco_probe_mfma, msco_probe_read) do what their headers say: the benchmark's
yardsticks rest on them, so their arithmetic and their coverage of the buffer are checked, not only their timing."""
import numpy as np
import pytest
import torch

from ms_custom_ops_amd import cabi

pytestmark = pytest.mark.gpu


def test_mfma_probe_multiplies_what_it_is_given():
    st = torch.cuda.current_stream().cuda_stream
    sink = torch.full((cabi.PROBE_MFMA_WORKGROUPS * 256,), -1, dtype=torch.int32, device="cuda:0")
    iters = 37
    # all ones: every round adds K = 32 to each of a lane's 256 accumulators; the sink holds their sum
    ones = torch.ones(cabi.PROBE_MFMA_OPERAND_BYTES, dtype=torch.int8, device="cuda:0")
    cabi.probe_mfma(ones.data_ptr(), sink.data_ptr(), iters, st)
    torch.cuda.synchronize()
    assert (sink.cpu().numpy() == 256 * 32 * iters).all()
    zeros = torch.zeros(cabi.PROBE_MFMA_OPERAND_BYTES, dtype=torch.int8, device="cuda:0")
    cabi.probe_mfma(zeros.data_ptr(), sink.data_ptr(), iters, st)
    torch.cuda.synchronize()
    assert (sink.cpu().numpy() == 0).all()
    with pytest.raises(cabi.BackendError):
        cabi.probe_mfma(0, sink.data_ptr(), iters, st)


@pytest.mark.parametrize("nbytes,wgs", [(4096 * 64, 8), (4096 * 1000 + 123, 7), (4096 * 3, 16)])
def test_read_probe_reads_every_byte_once(nbytes, wgs):
    # the xor of everything a workgroup's threads report is the xor of all dwords of the workgroup's share
    st = torch.cuda.current_stream().cuda_stream
    rng = np.random.default_rng(nbytes)
    host = rng.integers(0, 2 ** 32, nbytes // 4 + 1, dtype=np.uint64).astype(np.uint32)
    buf = torch.from_numpy(host.view(np.int32)).to("cuda:0")
    sink = torch.zeros(wgs * 256, dtype=torch.int32, device="cuda:0")
    cabi.probe_read(buf.data_ptr(), nbytes, sink.data_ptr(), wgs, st)
    torch.cuda.synchronize()
    got = np.bitwise_xor.reduce(sink.cpu().numpy().view(np.uint32))
    steps = nbytes // 4096
    want = np.bitwise_xor.reduce(host[:steps * 1024]) if steps else np.uint32(0)
    assert got == want
