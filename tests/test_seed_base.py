"""Host-side checks of the device seed base (the offset the gradient quantizers read at run time, for training steps
replayed from a captured graph): argument validation only; what the kernels do with it is tested on the GPU."""
import pytest
import torch

import quartet_amd
from quartet_amd import linear


def test_seed_base_must_be_an_int64_tensor_on_the_gpu():
    assert linear._SEED_BASE is None
    with pytest.raises(ValueError):
        quartet_amd.set_device_seed_base(torch.zeros(1, dtype=torch.int64))          # on the CPU
    with pytest.raises(ValueError):
        quartet_amd.set_device_seed_base(torch.zeros(1, dtype=torch.int32))
    assert linear._SEED_BASE is None
    quartet_amd.set_device_seed_base(None)
    assert linear._SEED_BASE is None


def test_the_seeded_entry_point_is_declared_and_exported():
    from quartet_amd import _lib
    assert "qm_linear_backward_seeded" in _lib.EXPORTS
    L = _lib.lib()
    assert L.qm_linear_backward_seeded.argtypes[:-2] == L.qm_linear_backward.argtypes[:-1]
