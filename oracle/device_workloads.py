"""Large synthetic CSR inputs built on the device.  TEST INFRASTRUCTURE (used by
bench.py and the full-size GPU tests): the host generator of
``oracle/workloads.py`` needs minutes at 4e8 non-zeros, the same construction
with PyTorch on the GPU takes a fraction of a second."""


def device_csr(torch, lengths_np, ncols, seed):
    """CSR structure with sorted distinct uniform columns per row, built on the
    device (the host generator of oracle/workloads.py needs minutes at 4e8
    non-zeros).  Returns (data f32, indptr i32, indices i32) device tensors."""
    dev = "cuda"
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    lengths = torch.from_numpy(lengths_np).to(dev)
    m = lengths.numel()
    indptr = torch.zeros(m + 1, dtype=torch.int64, device=dev)
    torch.cumsum(lengths, 0, out=indptr[1:])
    nnz = int(indptr[-1].item())
    assert nnz < 2**31
    row_of = torch.repeat_interleave(torch.arange(m, device=dev, dtype=torch.int64), lengths)
    cols = torch.randint(0, ncols, (nnz,), generator=g, device=dev, dtype=torch.int64)
    for _ in range(64):
        key = row_of * ncols + cols
        sk, order = torch.sort(key)
        dup_sorted = torch.zeros(nnz, dtype=torch.bool, device=dev)
        dup_sorted[1:] = sk[1:] == sk[:-1]
        ndup = int(dup_sorted.sum().item())
        if ndup == 0:
            cols = sk % ncols
            break
        idx = order[dup_sorted]
        cols[idx] = torch.randint(0, ncols, (ndup,), generator=g, device=dev, dtype=torch.int64)
        del key, sk, order, dup_sorted, idx
    else:
        raise RuntimeError("could not draw distinct columns")
    data = torch.randn(nnz, generator=g, device=dev, dtype=torch.float32)
    return data, indptr.to(torch.int32), cols.to(torch.int32)
