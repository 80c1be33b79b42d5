"""scatter_nd through the torch op and the C ABI against the CPU oracle.  Shapes follow
tests/python/test_scatter_nd.py (data [7,8,9,10], 5 index rows of depth 2, three dtypes); unlike
that test the tensors keep their shapes and the expectation is accumulation, which is what the
reference kernel computes."""

import pytest
import torch

from oracle import numerics as N

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("depth", [1, 2, 4])
def test_scatter_nd_accumulates(dtype, depth):
    from tilefusion_amd.ops import scatter_nd
    g = torch.Generator().manual_seed(1234 + depth)
    shape = [7, 8, 9, 10]
    data = torch.full(shape, 5.0, dtype=dtype)
    rows = 5 if depth < 4 else 300
    idx = torch.stack([torch.randint(0, shape[j], (rows,), generator=g) for j in range(depth)], dim=1)
    idx[1] = idx[0]                                               # a duplicate row must accumulate
    upd = torch.randint(-4, 5, (rows, *shape[depth:]), generator=g).to(dtype)   # small integers: exact in bf16
    want = N.scatter_nd_ref(data, idx, upd)
    dev = data.to(DEV)
    scatter_nd(dev, idx.to(DEV), upd.to(DEV))
    assert torch.equal(dev.float().cpu(), want)


def test_out_of_range_rows_are_skipped_and_shapes_checked():
    from tilefusion_amd.ops import scatter_nd
    data = torch.zeros(4, 6, device=DEV)
    idx = torch.tensor([[1], [9], [-1], [3]], device=DEV)
    upd = torch.ones(4, 6, device=DEV)
    scatter_nd(data, idx, upd)
    assert data.sum().item() == 12 and data[1].sum().item() == 6 and data[3].sum().item() == 6
    with pytest.raises(RuntimeError, match="updates must hold"):
        scatter_nd(data, idx, torch.ones(3, 6, device=DEV))
    with pytest.raises(RuntimeError, match="int64"):
        scatter_nd(data, idx.int(), upd)
