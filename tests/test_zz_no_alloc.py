"""The allocation-free entry point tsne_hip_max_normalize_noalloc against
tsne_hip_max_normalize, through the C ABI: bit-identical results on two calls in
a row (the second on a smaller input, so that nothing of the first call's
scratch contents may leak into it), and the size limit."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def test_max_normalize_noalloc_matches_allocating_entry_point():
    from tsnecuda import stages
    stages.lib()
    rng = np.random.default_rng(11)
    first = (rng.standard_normal(3_000_017) * 7.5).astype(np.float32)
    second = (rng.standard_normal(40_961) * 0.25).astype(np.float32)  # smaller input, smaller maximum
    assert np.abs(second).max() < np.abs(first).max()
    for values in (first, second):
        want = stages.max_normalize_(torch.from_numpy(values.copy()).cuda()).cpu().numpy()
        dev = torch.from_numpy(values.copy()).cuda()
        stages.max_normalize_noalloc_(dev)
        torch.cuda.synchronize()
        got = dev.cpu().numpy()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        np.testing.assert_array_equal(want, values / np.abs(values).max())


def test_max_normalize_noalloc_rejects_sizes_beyond_its_limit():
    from tsnecuda import stages
    stages.lib()
    dev = torch.ones(16, dtype=torch.float32, device="cuda")
    with pytest.raises(RuntimeError, match="exceed the supported maximum"):
        stages.max_normalize_noalloc_(dev, n=(1 << 32) + 1)
    torch.cuda.synchronize()
    assert torch.all(dev == 1.0)
