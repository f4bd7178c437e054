"""sddmm_csr_noalloc (the entry point that allocates nothing) against the plan-based
row-gather path it is a variant of: same kernel, so the outputs must agree bit for bit.
Two calls in a row share the library's one device array, the second on a smaller input.
The allocation check looks at the steady state (the second call): the first call of a process
on a device is where the runtime may load the code object and materialise the fixed array."""
import gc

import numpy as np
import pytest
import torch

from sddmm_gpu_amd import capi, synth

pytestmark = pytest.mark.gpu


def plan_based(dd, d, K, with_val):
    plan = capi.Plan.from_device_csr(d["n_rows"], d["n_cols"], d["nnz"], dd["row_ptr"].data_ptr(), dd["col_ind"].data_ptr(),
                                     K, 0, 0, capi.KERNEL_ROW_GATHER)
    out = torch.full((d["nnz"],), float("nan"), device=dd["W"].device)
    plan.execute(dd["val"].data_ptr() if with_val else 0, dd["W"].data_ptr(), dd["H"].data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    plan.close()
    return out


def no_alloc(dd, d, K, with_val):
    out = torch.full((d["nnz"],), float("nan"), device=dd["W"].device)
    stream = torch.cuda.current_stream().cuda_stream

    def call():
        capi.csr_noalloc(d["n_rows"], d["n_cols"], d["nnz"], dd["row_ptr"].data_ptr(), dd["col_ind"].data_ptr(),
                         dd["val"].data_ptr() if with_val else 0, K, dd["W"].data_ptr(), dd["H"].data_ptr(), out.data_ptr(), stream)
        torch.cuda.synchronize()

    # Device memory the driver reports free: a hipMalloc inside the call (by the library or by anything it calls)
    # would lower it.  The first launch of a kernel in a process lets the HIP runtime load code and set up its own
    # buffers, so the figure is taken around a second, identical call.  (Python garbage of earlier tests is
    # collected first, so that nothing is released meanwhile; torch keeps what it frees in its own cache, which
    # does not change the driver's figure.)
    call()
    first = out.clone()
    out.fill_(float("nan"))
    gc.collect()
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    call()
    assert torch.cuda.mem_get_info()[0] >= free_before
    assert torch.equal(out, first)
    return out


def to_dev(d):
    dev = torch.device("cuda:0")
    return {k: (v.to(dev).contiguous() if torch.is_tensor(v) else v) for k, v in d.items()}


def test_two_calls_second_smaller(oracle):
    big = synth.make(3, 0.02, K=128)      # power-law rows, many of them empty or of one nonzero
    small = synth.make(1, 0.25, K=128)    # a smaller, uniform matrix: its batches overwrite only a prefix of the array
    assert small["nnz"] < big["nnz"]
    for d in (big, small):
        dd = to_dev(d)
        want = plan_based(dd, d, 128, True)
        got = no_alloc(dd, d, 128, True)
        assert torch.equal(got, want), int((got != want).sum())
        cpu = oracle.sddmm_csr(d["row_ptr"].numpy(), d["col_ind"].numpy(), d["val"].numpy(), d["W"].numpy(), d["H"].numpy())
        _, absp = oracle.sddmm_f64(d["row_ind"].numpy(), d["col_ind"].numpy(), d["val"].numpy(), d["W"].numpy(), d["H"].numpy())
        bad = np.abs(got.cpu().numpy() - cpu) > 1e-5 * np.sqrt(128) * np.maximum(np.abs(cpu), absp / 100.0)
        assert not bad.any(), int(bad.sum())


@pytest.mark.parametrize("K,with_val", [(32, True), (64, False), (100, True), (30, True), (512, True)])
def test_other_ranks_and_no_values(K, with_val):
    d = synth.make(2, 0.3, K=K)
    dd = to_dev(d)
    want = plan_based(dd, d, K, with_val)
    got = no_alloc(dd, d, K, with_val)
    assert torch.equal(got, want), int((got != want).sum())


def test_empty_rows_and_empty_matrix():
    dev = torch.device("cuda:0")
    # rows 0, 2, 3 and the last two are empty; row 1 spans more than one batch of 64
    counts = [0, 150, 0, 0, 1, 63, 2, 0, 0]
    n_rows, n_cols, K = len(counts), 200, 64
    g = torch.Generator().manual_seed(7)
    cols = torch.cat([torch.randperm(n_cols, generator=g)[:c].sort().values for c in counts]).to(torch.int32)
    row_ptr = torch.tensor([0] + list(np.cumsum(counts)), dtype=torch.int32)
    d = dict(n_rows=n_rows, n_cols=n_cols, nnz=int(cols.numel()), row_ptr=row_ptr, col_ind=cols,
             val=torch.rand(cols.numel(), generator=g) + 0.5, W=torch.randn(n_rows, K, generator=g), H=torch.randn(n_cols, K, generator=g))
    dd = to_dev(d)
    assert dd["W"].device == dev
    want = plan_based(dd, d, K, True)
    got = no_alloc(dd, d, K, True)
    assert torch.equal(got, want)
    # nothing to do, nothing touched
    capi.csr_noalloc(5, 5, 0, 0, 0, 0, 8, 0, 0, 0)


def test_rejects_sizes_beyond_the_fixed_array():
    with pytest.raises(capi.SddmmError) as e:
        capi.csr_noalloc(10, 10, (1 << 28) + 1, 8, 8, 0, 8, 16, 16, 16)
    assert e.value.code == capi.ERR_RANGE
    # nonzeros in a matrix without rows: refused on the host, nothing is launched
    with pytest.raises(capi.SddmmError) as e:
        capi.csr_noalloc(0, 10, 5, 8, 8, 0, 8, 16, 16, 16)
    assert e.value.code == capi.ERR_ARG
