"""Small imperative programs (views, in-place writes, loops, branches) through the
whole route on the GPU: script -> build -> regions run by tssa::ParallelFunctor,
everything that is not a region by ATen on the device.  Reference: eager PyTorch on
the CPU.  The programs are the ones of tests/test_tensorssa.py."""
import pytest
import torch

import functs_amd.jit as fj
from tests.test_tensorssa import PROGRAMS, _IDS, _clone

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("fn,make", PROGRAMS, ids=_IDS)
def test_program_on_gpu(fn, make):
    gen = torch.Generator().manual_seed(4321)
    args = make(gen)
    want = fn(*_clone(args))
    built = fj.build(fj.script(fn, add_clone=True), list(args))
    dev_args = [a.cuda() if isinstance(a, torch.Tensor) else a for a in args]
    got = built(*dev_args)
    torch.testing.assert_close(got.cpu(), want, rtol=1e-5, atol=1e-6)
    # a second call reuses the compiled variants and must not see state of the first
    got2 = built(*dev_args)
    assert torch.equal(got2, got)
