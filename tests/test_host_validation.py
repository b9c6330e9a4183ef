"""Host-side contract of the Python entry points, checked without a GPU the way the reference tests
its dispatcher without hardware (backends/_enflame/test/test_sage_attention_native.py:240-293):
error classes follow backends/_hygon/ops/sageattention/sageattention_hip.py:30-74 and
backends/_enflame/ops/sage_attention/attn_qk_int8_per_block_native.py:212-276."""
import pytest
import torch

import baselinebenchmark_amd as sa
from baselinebenchmark_amd import sageattention as S


class FakeGpu(torch.Tensor):
    """A CPU tensor that claims to be on the GPU, so that shape/dtype checks can be reached."""

    @property
    def is_cuda(self):
        return True


def fake(*shape, dtype=torch.float16):
    return torch.zeros(shape, dtype=dtype).as_subclass(FakeGpu)


def test_cpu_tensors_are_rejected():
    x = torch.zeros((1, 2, 128, 64), dtype=torch.float16)
    with pytest.raises(TypeError):
        sa.per_block_int8(x, x)
    with pytest.raises(TypeError):
        sa.sageattn(x, x, x)
    with pytest.raises(TypeError):
        sa.forward(x.to(torch.int8), x.to(torch.int8), x, torch.zeros(1), torch.zeros(1))


def test_per_block_int8_contract():
    with pytest.raises(TypeError):
        sa.per_block_int8(fake(1, 2, 128, 64, dtype=torch.float32), fake(1, 2, 128, 64))
    with pytest.raises(ValueError):
        sa.per_block_int8(fake(2, 128, 64), fake(2, 128, 64))  # rank 3
    with pytest.raises(ValueError):
        sa.per_block_int8(fake(1, 2, 128, 64), fake(1, 2, 128, 64, dtype=torch.bfloat16))
    with pytest.raises(NotImplementedError):
        sa.per_block_int8(fake(1, 2, 128, 96), fake(1, 2, 128, 96))
    with pytest.raises(NotImplementedError):
        sa.per_block_int8(fake(1, 2, 128, 64), fake(1, 2, 128, 64), BLKQ=100)
    with pytest.raises(ValueError):
        sa.per_block_int8(fake(1, 2, 128, 64), fake(1, 2, 128, 64), tensor_layout="DNH")
    with pytest.raises(ValueError):
        sa.per_block_int8(fake(1, 2, 128, 64).transpose(1, 2), fake(1, 2, 128, 64))  # not contiguous


def test_forward_contract():
    q = fake(1, 4, 128, 64, dtype=torch.int8)
    k = fake(1, 2, 128, 64, dtype=torch.int8)
    v = fake(1, 2, 128, 64)
    qs, ks = fake(1, 4, 1, dtype=torch.float32), fake(1, 2, 2, dtype=torch.float32)
    with pytest.raises(TypeError):
        sa.forward(q.to(torch.int16).as_subclass(FakeGpu), k, v, qs, ks)
    with pytest.raises(TypeError):
        sa.forward(q, k, v, qs.half().as_subclass(FakeGpu), ks)
    with pytest.raises(NotImplementedError):
        sa.forward(q, k, v, qs, ks, output_dtype=torch.float32)
    with pytest.raises(ValueError):
        sa.forward(q, k, v, qs, ks, maxnreg=0)
    with pytest.raises(NotImplementedError):   # an explicit mask and the causal flag exclude each other
        sa.forward(q, k, v, qs, ks, attn_mask=fake(1, 4, 128, 128, dtype=torch.bool), is_causal=True)
    with pytest.raises(ValueError):             # mask on another device
        sa.forward(q, k, v, qs, ks, attn_mask=torch.ones(1, 4, 128, 128, dtype=torch.bool))
    with pytest.raises(ValueError):             # not broadcastable to [B, Hq, Sq, Skv]
        sa.forward(q, k, v, qs, ks, attn_mask=fake(1, 4, 128, 100, dtype=torch.bool))
    with pytest.raises(TypeError):              # neither boolean nor floating point
        sa.forward(q, k, v, qs, ks, attn_mask=fake(1, 4, 128, 128, dtype=torch.int32))
    with pytest.raises(ValueError):
        sa.forward(q, k, fake(1, 2, 64, 64), qs, ks)  # v length differs
    with pytest.raises(ValueError):
        sa.forward(fake(1, 3, 128, 64, dtype=torch.int8), k, v, fake(1, 3, 1, dtype=torch.float32), ks)  # 3 % 2
    with pytest.raises(ValueError):
        sa.forward(q, k, v, fake(1, 4, 2, dtype=torch.float32), ks)  # q_scale shape
    with pytest.raises(NotImplementedError):
        sa.forward(q, k, v, qs, ks, BLKK=8)
    with pytest.raises(ValueError):
        sa.forward(q, k, v, qs, ks, tensor_layout="XYZ")


def test_sageattn_contract():
    q, k = fake(1, 128, 4, 128), fake(1, 128, 2, 128)
    with pytest.raises(NotImplementedError):
        sa.sageattn(q, k, k, tensor_layout="NHD", qk_quant_dtype="fp8")
    with pytest.raises(ValueError):
        sa.sageattn(q, k, fake(1, 64, 2, 128), tensor_layout="NHD")
    with pytest.raises(ValueError):
        sa.sageattn(q, k, k, tensor_layout="NHD", pv_mode="int4")
    with pytest.raises(TypeError):
        sa.sageattn(q, k, k, tensor_layout="NHD", bogus=1)
    with pytest.raises(ValueError):
        sa.sageattn(fake(1, 128, 3, 128), k, k, tensor_layout="NHD")
    # quant_recipe as passed at sage_attention_benchmark_compare.py:300-313: (Q rows, K rows, -1, 1) -> FP8 V
    with pytest.raises(ValueError):
        sa.sageattn(q, k, k, tensor_layout="NHD", quant_recipe=(128, 16))
    with pytest.raises(NotImplementedError):
        sa.sageattn(q, k, k, tensor_layout="NHD", quant_recipe=(128, 16, 64, 1))
    with pytest.raises(ValueError):
        sa.sageattn(q, k, k, tensor_layout="NHD", quant_recipe=(128, 16, -1, 1), pv_mode="fp16")
    with pytest.raises(NotImplementedError):
        sa.sageattn(q, k, k, tensor_layout="NHD", quant_recipe=(128, 8, -1, 1))      # K blocks: 16 rows or more


def test_varlen_contract():
    q, k = fake(300, 4, 128), fake(300, 2, 128)
    cu = torch.tensor([0, 100, 300], dtype=torch.int32)
    with pytest.raises(ValueError):
        sa.sageattn_varlen(fake(1, 300, 4, 128), k, k, cu, cu, 200, 200)
    with pytest.raises(TypeError):
        sa.sageattn_varlen(q, k, k, cu.long(), cu, 200, 200)
    with pytest.raises(ValueError):
        sa.sageattn_varlen(q, k, k, cu, cu[:2], 200, 200)


def test_backend_name_is_a_function():
    # backends/_hygon/ops/sageattention/sageattention_hip.py:77-79
    assert callable(sa.backend_name) and isinstance(sa.backend_name(), str)


def test_q_multiplier_is_the_reference_double_product():
    assert S._q_mult(128, None) == 128 ** -0.5 * 1.44269504
    assert S._q_mult(64, 0.2) == 0.2 * 1.44269504
