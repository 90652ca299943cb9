"""The kernels' status word reaches the caller: bit 1 (a partial sum of a split K dimension did not
arrive; the output is invalid) becomes an exception and the workspace is cleared, bit 0 (a delta id
out of range, served as "no delta") a warning.  The reference reports every failure of its ops as a
Python exception (serving/vllm/delta/models.py:341-342, quant_linear_naive.py:19-20).

No kernel is made to fail here: the status word is set by hand."""
import warnings

import pytest
import torch

from deltazip_amd import ops


def test_status_word_meaning():
    ops._warned_bad_id = False
    ops.raise_for_status(0)
    with pytest.raises(ops.DeltaKernelError, match="partial sum .* did not arrive"):
        ops.raise_for_status(ops.STATUS_SUM_MISSING)
    with pytest.raises(RuntimeError, match="invalid"):          # a RuntimeError, like DZ_ELAUNCH
        ops.raise_for_status(ops.STATUS_SUM_MISSING | ops.STATUS_BAD_ID, "o_proj")
    with pytest.warns(RuntimeWarning, match="delta id outside"):
        ops.raise_for_status(ops.STATUS_BAD_ID)
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        ops.raise_for_status(ops.STATUS_BAD_ID)                   # once per process
    ops._warned_bad_id = False


@pytest.mark.gpu
def test_poll_status_raises_and_clears(dev):
    ops._warned_bad_id = False
    ws = ops._workspace(dev, 32, 4096, 4096)
    torch.cuda.synchronize()
    ops.poll_status(dev, wait=True)                               # clean
    # a failed exchange, as the kernel would leave it: bit 1 and a slot that is not empty
    ws[:4].view(torch.int32).fill_(ops.STATUS_SUM_MISSING)
    ws[8192:8196].view(torch.int32).fill_(0x3f800000)
    ops.poll_status(dev)                                          # starts the copy, nothing to look at yet
    torch.cuda.synchronize()
    with pytest.raises(ops.DeltaKernelError):
        ops.poll_status(dev)                                      # the copy of the previous call is in
    torch.cuda.synchronize()
    assert int(ws[:4].view(torch.int32).item()) == 0
    assert int(ws[256:].view(torch.int32).abs().sum().item()) == 0    # the slots are empty again
    ops.poll_status(dev, wait=True)
    # an id out of range: a warning, once
    ws[:4].view(torch.int32).fill_(ops.STATUS_BAD_ID)
    with pytest.warns(RuntimeWarning):
        ops.poll_status(dev, wait=True)
    assert ops.workspace_status() == 0
    ops._warned_bad_id = False


@pytest.mark.gpu
def test_status_word_survives_a_larger_workspace(dev):
    ws = ops._workspace(dev, 32, 4096, 4096)
    ws[:4].view(torch.int32).fill_(ops.STATUS_BAD_ID)
    big = ops._workspace(dev, 32, 4096, 16 * ws.numel() // 2048)   # needs more room: a new buffer
    assert big.data_ptr() != ws.data_ptr()
    assert ops.workspace_status() == ops.STATUS_BAD_ID
    big[:4].zero_()
