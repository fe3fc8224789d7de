"""Helpers shared by the GPU parity tests: device buffers come from torch (plumbing only), every
computation under test goes through the C ABI of libcct_hip.so."""
import numpy as np

_state = {}


def driver():
    """One HIPDriver per test process, bound to torch's current stream."""
    if "drv" not in _state:
        import torch
        from caffecontroll_amd import HIPDriver
        assert torch.cuda.is_available(), "GPU tests need a GPU"
        torch.cuda.init()
        drv = HIPDriver(0)
        drv.set_stream(torch.cuda.current_stream().cuda_stream)
        _state["drv"] = drv
    return _state["drv"]


class tuning:
    """`with tuning("direct_tile", 22): ...` pins a library tuning knob and puts `default` back after."""

    def __init__(self, name, value, default=0):
        self.name, self.value, self.default = name, value, default

    def __enter__(self):
        driver().set_tuning(self.name, self.value)

    def __exit__(self, *exc):
        driver().set_tuning(self.name, self.default)


def dev(a, dtype=None):
    import torch
    t = torch.from_numpy(np.ascontiguousarray(a if dtype is None else a.astype(dtype)))
    return t.cuda()


def empty(shape, dtype=None, fill=None):
    import torch
    dtype = dtype or torch.float32
    if fill is None:
        # poison so that unwritten elements are noticed
        t = torch.full(shape, float("nan"), dtype=dtype, device="cuda") if dtype.is_floating_point \
            else torch.full(shape, -7, dtype=dtype, device="cuda")
    else:
        t = torch.full(shape, fill, dtype=dtype, device="cuda")
    return t


def host(t):
    import torch
    torch.cuda.synchronize()
    return t.detach().cpu().numpy()


def rel_err(got, ref):
    """max|got-ref| / max|ref| -- the normalisation used for every fp32 tolerance in these tests."""
    ref = np.asarray(ref, np.float64)
    got = np.asarray(got, np.float64).reshape(ref.shape)
    denom = np.abs(ref).max()
    return np.abs(got - ref).max() / (denom if denom > 0 else 1.0)
