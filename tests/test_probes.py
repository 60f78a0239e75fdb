"""The two measurement aids of the C ABI (msco_probe_mfma_issue, msco_probe_read) do what their headers say: the benchmark's
yardsticks rest on them, so their arithmetic and their coverage of the buffer are checked, not only their timing."""
import numpy as np
import pytest
import torch

from ms_custom_ops_amd import cabi

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("pattern", [0, 8, 12, 13])
def test_mfma_probe_multiplies_what_it_is_given(pattern):
    st = torch.cuda.current_stream().cuda_stream
    sink = torch.full((cabi.PROBE_MFMA_WORKGROUPS * 256,), -1, dtype=torch.int32, device="cuda:0")
    clocks = torch.zeros(2, dtype=torch.int64, device="cuda:0")
    iters = 40
    # all ones: a round adds 64 blocks x 4 accumulators x K = 64 (16 blocks x 16 x K = 32, twice) to a thread's sum, whatever
    # memory operations are woven in
    ones = torch.ones(cabi.PROBE_MFMA_OPERAND_BYTES, dtype=torch.int8, device="cuda:0")
    cabi.probe_mfma_issue(ones.data_ptr(), sink.data_ptr(), clocks.data_ptr(), pattern, iters, st)
    torch.cuda.synchronize()
    assert (sink.cpu().numpy() == 16384 * iters).all()
    c = clocks.cpu().numpy()
    assert c[0] >= iters * 1000 and c[1] > 0   # 64 MFMAs of 16 cycles (32 of 32) per round at least
    zeros = torch.zeros(cabi.PROBE_MFMA_OPERAND_BYTES, dtype=torch.int8, device="cuda:0")
    cabi.probe_mfma_issue(zeros.data_ptr(), sink.data_ptr(), clocks.data_ptr(), pattern, iters, st)
    torch.cuda.synchronize()
    assert (sink.cpu().numpy() == 0).all()
    with pytest.raises(cabi.BackendError):
        cabi.probe_mfma_issue(0, sink.data_ptr(), clocks.data_ptr(), pattern, iters, st)
    with pytest.raises(cabi.BackendError):
        cabi.probe_mfma_issue(ones.data_ptr(), sink.data_ptr(), clocks.data_ptr(), 99, iters, st)
    with pytest.raises(cabi.BackendError):
        cabi.probe_mfma_issue(ones.data_ptr(), sink.data_ptr(), clocks.data_ptr(), pattern, 37, st)   # rounds come in eights


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
