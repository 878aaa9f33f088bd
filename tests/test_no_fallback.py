"""There is no CPU path and no silent fallback: host tensors are refused, and a kernel library
that is missing and cannot be compiled is an error that carries the compiler's output."""
import pytest
import torch

from rocml_amd import ops
from rocml_amd.csrc import build
from rocml_amd.errors import ExtensionMissingError, KernelError


def test_host_tensors_are_refused():
    x = torch.zeros(2, 8)
    gain = torch.ones(8)
    out = torch.empty(2, 8)
    with pytest.raises(KernelError, match="no CPU path"):
        ops.rmsnorm(x, gain, 1e-6, out)
    with pytest.raises(KernelError, match="no CPU path"):
        ops.gemm(x, torch.zeros(4, 8), torch.empty(2, 4))
    ids = torch.zeros(2, dtype=torch.int32)
    with pytest.raises(KernelError, match="no CPU path"):
        ops.embed_gather(torch.zeros(5, 8), ids, out)


def test_a_library_that_cannot_be_built_is_an_error(tmp_path, monkeypatch):
    # a checkout without built libraries and a compiler that fails
    monkeypatch.setattr(build, "SRC_DIR", str(tmp_path))
    monkeypatch.setenv("HIPCC", "/bin/false")
    with pytest.raises(ExtensionMissingError, match="hipcc failed for attention.hip"):
        build.ensure("attention")
    assert not (tmp_path / "_build" / "libattention.so").exists()
    with pytest.raises(ExtensionMissingError, match="unknown kernel family"):
        build.build(["nothing"], force=False)
