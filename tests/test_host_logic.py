"""Host-side mirror (prism_amd.ops) checks that need no GPU: argument validation
and the error behaviour taken over from the reference's launchers."""
import pytest
import torch

import prism_amd
from prism_amd import ops


def test_unknown_kernel_number_raises_like_the_reference():
    # run_my_kernel: `default: throw std::invalid_argument("Unknown my_kernel number")`
    # (evals/4090_sgemm/runner.cu:263-266)
    for bad in (0, 6, 7, -3):
        with pytest.raises(ValueError, match="Unknown my_kernel number"):
            prism_amd.run_my_kernel(bad, 4, 4, 4, 1.0, 0, 0, 0.0, 0)
    with pytest.raises(ValueError, match="Unknown my_kernel number"):
        z = torch.zeros(16)
        prism_amd.sgemm(4, 4, 4, 1.0, z, z, 0.0, z, variant=9)


def test_host_tensors_are_rejected_not_computed_on_cpu():
    x = torch.zeros(16, dtype=torch.int32)
    with pytest.raises(ValueError, match="device memory"):
        prism_amd.add_m(x, torch.empty_like(x), 7)
    with pytest.raises(ValueError, match="device memory"):
        prism_amd.scan(x)
    a = torch.zeros(16, dtype=torch.float32)
    with pytest.raises(ValueError, match="device memory"):
        prism_amd.sgemm(4, 4, 4, 1.0, a, a, 0.0, a)
    h = torch.zeros((4, 8), dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="device memory"):
        prism_amd.gemm_bf16(h, h)


def test_dtype_and_size_checks():
    x = torch.zeros(16, dtype=torch.int64)
    with pytest.raises(TypeError):
        prism_amd.add_m(x, x, 7)
    with pytest.raises(TypeError):
        prism_amd.scan(torch.zeros(4, dtype=torch.float32))
    a = torch.zeros(15, dtype=torch.float32)
    with pytest.raises(ValueError, match="elements"):
        prism_amd.sgemm(4, 4, 4, 1.0, a, a, 0.0, a)
    with pytest.raises(ValueError, match="MxK"):
        prism_amd.gemm_bf16(torch.zeros((4, 8), dtype=torch.bfloat16), torch.zeros((4, 16), dtype=torch.bfloat16))


def test_workspace_size_mirror():
    assert prism_amd.get_workspace_size(0) > 0
    assert prism_amd.get_workspace_size(1 << 24) >= prism_amd.get_workspace_size(1 << 20)
    with pytest.raises(ValueError):
        prism_amd.get_workspace_size(-1)
    with pytest.raises(ValueError, match="workspace"):
        prism_amd.launch_scan(1 << 20, torch.zeros(1 << 20, dtype=torch.int32), torch.zeros(8, dtype=torch.uint8))


def test_kernel_table_matches_header():
    assert sorted(ops.SGEMM_KERNELS) == [1, 2, 3, 4, 5, 6]
    assert prism_amd.tile_coords(0, 4, 4) == (0, 0)
