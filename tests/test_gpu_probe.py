"""The read-only probe launch: it must read every 16-byte chunk of every row it is given."""
import numpy as np
import pytest
import torch

import lily_sampler as LS

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rows,cols", [(1, 4), (3, 4096 + 4), (40, 75_968)])
def test_probe_read_returns_each_rows_largest_word(rows, cols):
    s = LS.Sampler(0)
    rng = np.random.default_rng(rows)
    x = rng.integers(0, 2**31 - 1, (rows, cols), dtype=np.int64).astype(np.int32)
    x[rows - 1, cols - 1] = 2**31 - 1          # the very last word must be seen
    x[0, 0] = 2**31 - 2
    t = torch.from_numpy(x).cuda()
    out = torch.zeros(rows, dtype=torch.int32, device="cuda")
    s.probe_read(t, out)
    s.synchronize()
    assert np.array_equal(out.cpu().numpy(), x.max(axis=1))
    s.close()


def test_probe_read_rejects_misaligned_rows():
    s = LS.Sampler(0)
    t = torch.zeros((2, 6), dtype=torch.int32, device="cuda")   # 24-byte rows
    out = torch.zeros(2, dtype=torch.int32, device="cuda")
    with pytest.raises(LS.SamplerError):
        s.probe_read(t, out)
    s.close()
