"""GPU test of the run-time compiled path: a descriptor outside the ahead-of-time
set is compiled with hiprtc, cached on disk, loaded and launched."""
import pytest
import torch

import kermac_amd as kermac
from kermac_amd.module_cache import module_cache as mc
from oracle import oracle
from tests.helpers import assert_close_to_truth

pytestmark = pytest.mark.gpu


def test_jit_descriptor_end_to_end(device, tmp_path, monkeypatch):
    monkeypatch.setenv("KERMAC_AMD_CACHE_DIR", str(tmp_path))
    mc.Singleton._instances.pop(mc.ModuleCache, None)
    try:
        # sum_k sqrt(b * a): DOT + SQRT is not compiled ahead of time
        desc = kermac.KernelDescriptor(kermac.InnerOperator.DOT, kermac.PowerType.SQRT, kermac.PowerType.SQUARE,
                                       kermac.KernelType.NONE)
        g = torch.Generator().manual_seed(5)
        a = torch.rand(150, 37, generator=g).to(device)
        b = torch.rand(3, 90, 37, generator=g).to(device)
        kermac.pre_compile_descriptors(device, [desc], try_to_align=True)
        assert len(list(tmp_path.glob("code-*.hsaco"))) == 1
        out = kermac.run_kernel(desc, a, b)
        truth = oracle.build_kernel("DOT", "SQRT", "SQUARE", "NONE", a.cpu(), b.cpu())
        assert_close_to_truth(out, truth, rtol=1e-5, what="jit DOT/SQRT/SQUARE")
        assert len(list(tmp_path.glob("code-*.hsaco"))) == 1          # nothing recompiled
        # column-major views pick another loader variant of the same descriptor
        out2 = kermac.run_kernel(desc, a.t().contiguous().t(), b)
        assert_close_to_truth(out2, truth, rtol=1e-5, what="jit, column-major a")
        # second process-wide cache instance: served from disk, then from memory
        mc.Singleton._instances.pop(mc.ModuleCache, None)
        out3 = kermac.run_kernel(desc, a, b)
        assert torch.equal(out3, out)
    finally:
        mc.Singleton._instances.pop(mc.ModuleCache, None)
