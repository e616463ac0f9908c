"""Shared plumbing of the GPU parity tests: device buffers with guard zones, calls through the C ABI."""
import numpy as np

import helpers

GUARD = 256  # elements of sentinel before and after every device tensor


class DeviceTensor:
    """A torch device buffer with sentinel guard zones on both sides of the payload."""

    def __init__(self, host):
        import torch
        self.n = host.size
        self.dtype = host.dtype
        full = np.full(self.n + 2 * GUARD, 777.0, dtype=host.dtype)
        full[GUARD:GUARD + self.n] = host
        self.t = torch.from_numpy(full).cuda()

    @property
    def ptr(self):
        return self.t.data_ptr() + GUARD * self.t.element_size()

    def host(self):
        return self.t.cpu().numpy()[GUARD:GUARD + self.n].copy()

    def guards_intact(self):
        full = self.t.cpu().numpy()
        return bool(np.all(full[:GUARD] == 777.0) and np.all(full[GUARD + self.n:] == 777.0))


def make_inputs(tools, expr, sizes, dtype, c_mode="seeded", seeds=(1, 2, 3)):
    nC, nA, nB = helpers.tensor_sizes(expr, sizes)
    A = tools.fill_uniform(np.empty(nA, dtype), seeds[0])
    B = tools.fill_uniform(np.empty(nB, dtype), seeds[1])
    C = tools.fill_uniform(np.empty(nC, dtype), seeds[2]) if c_mode == "seeded" else np.zeros(nC, dtype)
    return C, A, B


def run_entry(ex, sizes, C, A, B, variant=None):
    """Upload, call sd_t_d2_fusion_ (or cogent_run with a variant), download; checks guards and status."""
    import torch
    dC, dA, dB = DeviceTensor(C), DeviceTensor(A), DeviceTensor(B)
    if variant is None:
        rc = ex.entry(sizes, dC.ptr, dA.ptr, dB.ptr)
    else:
        rc = ex.run(sizes, dC.ptr, dA.ptr, dB.ptr, None, variant)
    torch.cuda.synchronize()
    assert rc == 0, "status %d: %s" % (rc, ex.last_error())
    assert dC.guards_intact(), "write outside C"
    assert np.array_equal(dA.host(), A) and np.array_equal(dB.host(), B), "inputs were modified"
    return dC.host()
