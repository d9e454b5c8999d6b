"""CPU checks of the host-side mirror of the reference interface: names, signatures, error behaviour, module state."""

import inspect

import pytest
import torch

import fma
from fma import KernelBackend, MoE, continuous_count, grouped_gemm, swiglu, swiglu_packed
from fma.ops.swiglu.cuda_implementation import _rows_view


def test_public_names_and_signatures():
    assert [b.value for b in KernelBackend] == ["cuda", "torch", "triton"]
    sig = inspect.signature(continuous_count)
    assert list(sig.parameters) == ["x", "size", "kernel_backend"]
    assert sig.parameters["kernel_backend"].kind is inspect.Parameter.KEYWORD_ONLY
    assert list(inspect.signature(grouped_gemm).parameters) == [
        "A", "B", "C", "M_array", "N_array", "K_array", "output_shape", "alpha", "beta", "is_A_transposed",
        "is_B_transposed", "benchmark",
    ]
    assert list(inspect.signature(swiglu).parameters) == ["gate", "up", "kernel_backend_forward", "kernel_backend_backward"]
    assert list(inspect.signature(swiglu_packed).parameters) == ["x", "kernel_backend_forward", "kernel_backend_backward"]
    assert list(inspect.signature(MoE.__init__).parameters)[1:] == [
        "num_experts", "num_experts_per_tok", "hidden_size", "intermediate_size", "activation_function", "is_glu",
        "add_bias", "std",
    ]
    assert inspect.signature(MoE.forward).parameters["kernel_backend"].default is KernelBackend.triton


def test_custom_ops_are_registered_with_reference_names():
    ns = torch.ops.flash_model_architectures
    for name in ["continuous_count_cuda", "grouped_gemm_cuda", "swiglu_forward_cuda", "swiglu_backward_cuda"]:
        assert hasattr(ns, name)


def test_module_state_dict_layout():
    moe = MoE(8, 2, 64, 128, swiglu_packed, True, False, 0.02)
    shapes = {k: tuple(v.shape) for k, v in moe.state_dict().items()}
    assert shapes == {
        "gate.weight": (8, 64),
        "c_fc.weight": (8, 256, 64),
        "c_fc.N_array": (8,),
        "c_fc.K_array": (8,),
        "c_proj.weight": (8, 64, 128),
        "c_proj.N_array": (8,),
        "c_proj.K_array": (8,),
    }
    assert moe.c_fc.N_array.dtype == torch.uint32 and moe.c_fc.N_array.tolist() == [256] * 8
    assert moe.c_proj.K_array.tolist() == [128] * 8
    assert moe.fuse_swiglu
    assert not MoE(8, 2, 64, 128, torch.nn.GLU(), True, False, 0.02).fuse_swiglu
    assert abs(float(moe.c_fc.weight.std()) - 0.02) < 2e-3


def test_unexpected_backends_raise():
    x = torch.zeros(4, dtype=torch.int64)
    with pytest.raises(ValueError, match="unexpected kernel_backend"):
        continuous_count(x, 8, kernel_backend=KernelBackend.torch)
    moe = MoE(4, 2, 16, 32, swiglu_packed, True, False, 0.02)
    with pytest.raises(ValueError, match="unexpected kernel_backend"):
        moe(torch.zeros(3, 16), kernel_backend=KernelBackend.torch)
    with pytest.raises(ValueError, match="unexpected kernel_backend"):
        swiglu(torch.zeros(2, 2), torch.zeros(2, 2), kernel_backend_forward=KernelBackend.torch)


def test_ops_refuse_cpu_tensors_instead_of_falling_back():
    with pytest.raises(RuntimeError, match="GPU only"):
        continuous_count(torch.zeros(4, dtype=torch.int64), 8)
    with pytest.raises(RuntimeError, match="GPU only"):
        swiglu(torch.zeros(2, 8), torch.zeros(2, 8))
    u32 = torch.zeros(2, dtype=torch.uint32)
    with pytest.raises(RuntimeError, match="GPU only"):
        grouped_gemm(torch.zeros(4, 8, dtype=torch.bfloat16), torch.zeros(4, 8, dtype=torch.bfloat16), None, u32, u32, u32, (4, 4))


def test_continuous_count_python_side_asserts():
    assert continuous_count(torch.zeros(5, dtype=torch.int64), 1).tolist() == [5]  # size == 1 shortcut, no kernel
    with pytest.raises(AssertionError):
        continuous_count(torch.zeros(2, 2, dtype=torch.int64), 8)
    with pytest.raises(AssertionError):
        continuous_count(torch.zeros(4, dtype=torch.int16), 8)
    with pytest.raises(AssertionError):
        grouped_gemm(None, None, None, None, None, None, (1,), beta=1)


def test_rows_view():
    x = torch.zeros(6, 10)
    assert _rows_view(x) == (6, 10, 10)
    up, gate = x.chunk(2, dim=-1)
    assert _rows_view(up) == (6, 5, 10) and _rows_view(gate) == (6, 5, 10)
    y = torch.zeros(2, 3, 8)
    assert _rows_view(y) == (6, 8, 8)
    assert _rows_view(y.chunk(2, -1)[1]) == (6, 4, 8)
    assert _rows_view(y.transpose(0, 1)) is None  # rows not equally spaced
    assert _rows_view(x.t()) is None  # last dim not contiguous
    assert _rows_view(torch.zeros(7)) == (1, 7, 7)


def test_package_has_no_oracle_dependency():
    import os

    root = os.path.dirname(fma.__file__)
    for dirpath, _, files in os.walk(root):
        for f in files:
            if f.endswith(".py"):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.replace("moe_oracle", "oracle") or "import oracle" not in text
                assert "from oracle" not in text and "import oracle" not in text


def test_fused_residual_add_rmsnorm_signature_and_errors():
    from fma import fused_residual_add_rmsnorm

    sig = inspect.signature(fused_residual_add_rmsnorm)
    assert list(sig.parameters) == ["x", "residual", "weight", "eps", "multiplier", "memory_efficient", "kernel_backend"]
    assert sig.parameters["multiplier"].default is None and sig.parameters["memory_efficient"].default is False
    assert sig.parameters["kernel_backend"].default is KernelBackend.triton
    x = torch.randn(4, 8)
    with pytest.raises(ValueError):
        fused_residual_add_rmsnorm(x, x, None, 1e-5, kernel_backend=KernelBackend.torch)
    with pytest.raises(RuntimeError, match="GPU only"):  # no eager implementation to fall back to
        fused_residual_add_rmsnorm(x, x, None, 1e-5)
    with pytest.raises(AssertionError, match="weight should be 1D"):
        fused_residual_add_rmsnorm(x, x, torch.randn(2, 8), 1e-5)
    with pytest.raises(AssertionError, match="hidden size"):
        fused_residual_add_rmsnorm(x, x, torch.randn(4), 1e-5)


def test_router_and_bias_host_logic():
    moe = MoE(8, 2, 64, 128, swiglu_packed, True, False, 0.02)
    assert moe.fuse_router and moe.fuse_swiglu and moe.c_fc.bias is None
    # the fused router serves 16-bit activations on the GPU only: everything else takes the reference's ATen formulation
    assert not moe._router_is_fusable(torch.randn(4, 64))
    assert not moe._router_is_fusable(torch.randn(4, 64).bfloat16())  # a CPU tensor
    logits, weights, selected = moe._compute_routing_weights(torch.randn(5, 64))
    assert logits.shape == (5, 8) and weights.shape == selected.shape == (5, 2) and selected.dtype == torch.int64
    assert torch.allclose(weights.sum(-1), torch.ones(5), atol=1e-6)
    assert bool((logits.gather(1, selected)[:, 0] >= logits.gather(1, selected)[:, 1]).all())
    # a layer with biases keeps them as parameters of the reference's shapes (the fused up-projection adds its own)
    biased = MoE(8, 2, 64, 128, swiglu_packed, True, True, 0.02)
    assert biased.c_fc.bias.shape == (8, 256) and biased.c_proj.bias.shape == (8, 64) and biased.fuse_swiglu
    assert float(biased.c_fc.bias.abs().max()) == 0.0  # reset_parameters zeroes them (fma/modules/moe/__init__.py:121-122)
    top1 = MoE(4, 1, 64, 128, swiglu_packed, True, False, 0.02)
    _, w1, s1 = top1._compute_routing_weights(torch.randn(5, 64))
    assert torch.equal(w1, torch.ones(5, 1)) and s1.shape == (5, 1)


def test_build_refuses_gemm_kernels_with_register_spills():
    # the grouped GEMM counts its outstanding memory operations by hand; the build reads the compiler's resource report
    # and fails when one of its kernels uses scratch memory (spill traffic would shift those counts)
    import build

    clean = "remark: Function Name: _Zfoo19grouped_gemm_kernelIbar\nremark:     ScratchSize [bytes/lane]: 0\n"
    build._check_no_scratch("grouped_gemm.hip", clean, "grouped_gemm_kernel")
    spilled = clean.replace("[bytes/lane]: 0", "[bytes/lane]: 24")
    with pytest.raises(RuntimeError, match="scratch"):
        build._check_no_scratch("grouped_gemm.hip", spilled, "grouped_gemm_kernel")
    with pytest.raises(RuntimeError, match="names no"):
        build._check_no_scratch("grouped_gemm.hip", "remark: Function Name: other\n", "grouped_gemm_kernel")
    assert "grouped_gemm.hip" in build.NO_SCRATCH_SOURCES
