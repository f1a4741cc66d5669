"""The counter-based input generator: numpy and torch must produce the same bits (torch on the CPU here;
the GPU tests regenerate windows of device buffers with numpy), and the distributions must be what
the benchmark claims."""
import numpy as np
import pytest

from megray_amd import synth

torch = pytest.importorskip("torch")

PAIRS = [(np.int8, torch.int8), (np.uint8, torch.uint8), (np.int32, torch.int32), (np.int64, torch.int64),
         (np.float16, torch.float16), (np.float32, torch.float32), (np.float64, torch.float64)]


@pytest.mark.parametrize("npdt,tdt", PAIRS)
def test_numpy_and_torch_agree_bit_for_bit(npdt, tdt):
    kinds = ("uniform", "normal") if np.dtype(npdt).kind == "f" and npdt != np.float64 else ("uniform",)
    for kind in kinds:
        for rank, start, count in ((0, 0, 1000), (5, (1 << 33) + 7, 4097), (15, 123, 1)):
            a = synth.fill_np(npdt, count, rank, kind, start)
            b = synth.fill_torch(tdt, count, rank, kind, start, device="cpu").numpy()
            assert a.dtype == b.dtype and np.array_equal(a.view(np.uint8), b.view(np.uint8)), (kind, rank, start)


def test_windows_are_consistent_and_ranks_differ():
    whole = synth.fill_np(np.float32, 5000, 3)
    assert np.array_equal(whole[1234:1300], synth.fill_np(np.float32, 66, 3, start=1234))
    assert not np.array_equal(whole, synth.fill_np(np.float32, 5000, 4))
    big = synth.fill_torch(torch.int32, (1 << 24) + 5, 1, device="cpu")  # crosses a generation slice
    assert np.array_equal(big[-9:].numpy(), synth.fill_np(np.int32, 9, 1, start=(1 << 24) - 4))


def test_distributions():
    u = synth.fill_np(np.float32, 1 << 20, 0)
    assert u.min() >= -1.0 and u.max() < 1.0 and abs(u.mean()) < 5e-3 and abs(u.var() - 1 / 3) < 5e-3
    d = synth.fill_np(np.float64, 1 << 18, 0)
    assert d.min() >= -1.0 and d.max() < 1.0 and np.unique(d).size > (1 << 18) - 8
    g = synth.fill_np(np.float32, 1 << 20, 2, "normal").astype(np.float64)
    assert abs(g.mean()) < 1e-4 and abs(g.std() - 0.01) < 2e-4
    assert abs(np.mean(np.abs(g) < 0.01) - 0.6827) < 0.01  # one sigma holds what a normal would
    i = synth.fill_np(np.int32, 1 << 20, 1)
    assert i.min() < -2 ** 30 and i.max() > 2 ** 30
    q = synth.fill_np(np.int64, 1 << 16, 1)
    assert q.min() < -2 ** 62 and q.max() > 2 ** 62
    b = synth.fill_np(np.uint8, 1 << 16, 1)
    assert np.bincount(b, minlength=256).min() > 150


def test_known_answers():
    # splitmix64's published first outputs for state 0 (the finaliser applied to GOLDEN, 2*GOLDEN, ...)
    # pin the mixing constants and shifts
    z = np.array([0, synth.GOLDEN], dtype=np.uint64)
    out = synth._mix_np(z)
    assert int(out[0]) == 0xE220A8397B1DCDAF and int(out[1]) == 0x6E789E6AA1B965F4
