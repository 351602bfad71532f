"""GPU parity of the RMSNorm (+ residual) and SiLU-and-multiply kernels against
the CPU oracle.  RMSNorm: bit-exact (kernel and oracle run the same IEEE fp32
sequence).  SiLU-and-multiply: the kernel evaluates in fp32, the oracle in
float64, so a result may differ by one bf16 ulp where the value sits on a
rounding boundary; the test allows that on at most 0.1 % of the elements."""
import numpy as np
import pytest

from helpers import bits_to_torch, torch_to_bits

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("T,hidden", [(128, 1024), (1, 8), (7, 520), (33, 4096), (5, 8192),
                                      (0, 1024)])
@pytest.mark.parametrize("with_residual", [False, True])
def test_add_rms_norm_bit_exact(T, hidden, with_residual):
    import torch
    from nanovllm_jax_amd.layers.layernorm import rms_norm
    from oracle.paged_attention_oracle import add_rms_norm_ref, f32_to_bf16_bits
    rng = np.random.Generator(np.random.PCG64(7000 + T + hidden))
    x = f32_to_bf16_bits(rng.standard_normal((T, hidden), dtype=np.float32) * 3)
    res = f32_to_bf16_bits(rng.standard_normal((T, hidden), dtype=np.float32) * 2)
    w = (1 + 0.3 * rng.standard_normal(hidden)).astype(np.float32)
    dev = "cuda:0"
    xt, wt = bits_to_torch(x, dev), torch.from_numpy(w).to(dev)
    if with_residual:
        rt = bits_to_torch(res, dev)
        y, new_res = rms_norm(xt, wt, 1e-6, rt, residual_out=rt)      # residual updated in place
        torch.cuda.synchronize()
        assert new_res is rt
        if T:
            want_y, want_r = add_rms_norm_ref(x, w, 1e-6, res)
            assert np.array_equal(torch_to_bits(new_res), want_r), "residual not bit-exact"
            assert np.array_equal(torch_to_bits(y), want_y), "output not bit-exact"
    else:
        y = rms_norm(xt, wt, 1e-6)
        torch.cuda.synchronize()
        if T:
            assert np.array_equal(torch_to_bits(y), add_rms_norm_ref(x, w, 1e-6))
    assert tuple(y.shape) == (T, hidden)


def test_rms_norm_class_mirrors_the_reference_call():
    import torch
    from nanovllm_jax_amd.layers.layernorm import RMSNorm
    from oracle.paged_attention_oracle import add_rms_norm_ref, f32_to_bf16_bits
    rng = np.random.Generator(np.random.PCG64(71))
    x = f32_to_bf16_bits(rng.standard_normal((2, 3, 256), dtype=np.float32))
    res = f32_to_bf16_bits(rng.standard_normal((2, 3, 256), dtype=np.float32))
    norm = RMSNorm(256, eps=1e-5, device="cuda:0")
    y = norm(bits_to_torch(x, "cuda:0"))
    y2, r2 = norm(bits_to_torch(x, "cuda:0"), bits_to_torch(res, "cuda:0"))
    torch.cuda.synchronize()
    ones = np.ones(256, np.float32)
    assert np.array_equal(torch_to_bits(y).reshape(6, 256),
                          add_rms_norm_ref(x.reshape(6, 256), ones, 1e-5))
    wy, wr = add_rms_norm_ref(x.reshape(6, 256), ones, 1e-5, res.reshape(6, 256))
    assert np.array_equal(torch_to_bits(y2).reshape(6, 256), wy)
    assert np.array_equal(torch_to_bits(r2).reshape(6, 256), wr)


@pytest.mark.parametrize("T,inter", [(128, 3072), (1, 8), (9, 40), (0, 64)])
def test_silu_and_mul(T, inter):
    import torch
    from nanovllm_jax_amd.layers.activation import silu_and_mul
    from oracle.paged_attention_oracle import (bf16_bits_to_f32, f32_to_bf16_bits,
                                               silu_and_mul_ref)
    rng = np.random.Generator(np.random.PCG64(7200 + T + inter))
    x = f32_to_bf16_bits(rng.standard_normal((T, 2 * inter), dtype=np.float32) * 4)
    if T:
        x[0, :4] = f32_to_bf16_bits(np.array([0.0, 80.0, -200.0, -1e30], np.float32))
    y = silu_and_mul(bits_to_torch(x, "cuda:0"))
    torch.cuda.synchronize()
    assert tuple(y.shape) == (T, inter)
    if not T:
        return
    got, want = torch_to_bits(y), silu_and_mul_ref(x)
    diff = got != want
    assert diff.mean() <= 1e-3
    # where they differ it is the neighbouring bf16 value
    assert np.all(np.abs(got[diff].astype(np.int32) - want[diff].astype(np.int32)) <= 1)
    assert not np.isnan(bf16_bits_to_f32(got)).any()


def test_layer_glue_argument_errors():
    import torch
    from nanovllm_jax_amd import _lib
    from nanovllm_jax_amd.layers.activation import silu_and_mul
    from nanovllm_jax_amd.layers.layernorm import rms_norm
    x = torch.zeros((2, 12), dtype=torch.bfloat16, device="cuda:0")
    w = torch.ones(12, dtype=torch.float32, device="cuda:0")
    with pytest.raises(_lib.NativeLibraryError):
        rms_norm(x, w, 1e-6)                       # hidden not a multiple of 8
    with pytest.raises(ValueError):
        rms_norm(x.float(), w, 1e-6)
    with pytest.raises(ValueError):
        silu_and_mul(x.cpu())
    with pytest.raises(_lib.NativeLibraryError):
        silu_and_mul(x)                            # intermediate 6 not a multiple of 8
