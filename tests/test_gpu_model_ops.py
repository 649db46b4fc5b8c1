"""The two elementwise launches of the decoder block around the attention path (SwiGLU on a merged gate / up
projection, residual add + RMS layer norm) against plain PyTorch fp32 references of the same formulas.

Tolerances: the result may differ from the fp32 reference by the roundings of the storage type (two for SwiGLU,
one for the norm, one for the residual sum): 1 ulp of bf16 / fp16 relative (2^-7 / 2^-10), 2e-6 for fp32."""
import pytest
import torch
import torch.nn.functional as F

from acache_amd import ops

pytestmark = pytest.mark.gpu
REL = {torch.bfloat16: 2 ** -7, torch.float16: 2 ** -10, torch.float32: 2e-6}


def _close(got, want, dtype, scale=1.0):
    err = (got.float() - want).abs()
    bound = REL[dtype] * (want.abs() + 1e-3) * scale
    assert (err <= bound).all(), float((err / (want.abs() + 1e-3)).max())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("M,m", [(1, 128), (37, 12288), (512, 128), (5, 8)])
def test_swiglu_matches_fp32_reference(device, dtype, M, m):
    g = torch.Generator(device=device).manual_seed(M + m)
    gu = (torch.randn(M, 2 * m, generator=g, device=device) * 2).to(dtype)
    got = ops.swiglu(gu, m)
    assert got.shape == (M, m) and got.dtype == dtype
    want = F.silu(gu[:, :m].float()) * gu[:, m:].float()
    _close(got, want, dtype, scale=1.05)
    # the separate kernels of the unmerged formulation round the same two times; an activation that rounds the
    # other way moves the product by at most one more ulp
    two_step = F.silu(gu[:, :m]) * gu[:, m:]
    _close(got, two_step.float(), dtype, scale=2.0)


def test_swiglu_on_a_batched_strided_projection(device):
    x = torch.randn(3, 8, 2 * 64 + 32, device=device).to(torch.bfloat16)[..., :128]      # rows wider than 2m
    got = ops.swiglu(x, 64)
    assert got.shape == (3, 8, 64)
    _close(got, F.silu(x[..., :64].float()) * x[..., 64:].float(), torch.bfloat16)
    with pytest.raises(ValueError):
        ops.swiglu(torch.zeros(4, 2 * 12, device=device, dtype=torch.bfloat16), 12)       # 24-byte halves


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("M,d", [(1, 64), (29, 4096), (512, 256), (3, 8192), (7, 3584)])
def test_add_rms_norm_matches_fp32_reference(device, dtype, M, d):
    g = torch.Generator(device=device).manual_seed(M + d)
    x = torch.randn(M, d, generator=g, device=device).to(dtype)
    delta = (torch.randn(M, d, generator=g, device=device) * 0.5).to(dtype)
    w = (1 + 0.1 * torch.randn(d, generator=g, device=device)).to(dtype)
    x0 = x.clone()
    if d * x.element_size() > 16384:                                 # rows of more than 16 KiB are refused
        with pytest.raises(ValueError):
            ops.add_rms_norm(x, delta, w, 1e-5)
        return
    total, y = ops.add_rms_norm(x, delta, w, 1e-5)
    assert torch.equal(x, x0)                                        # nothing modified in place
    assert torch.equal(total, x + delta)                             # the residual stream keeps the rounded sum
    s = total.float()
    want = s * torch.rsqrt(s.pow(2).mean(-1, keepdim=True) + 1e-5) * w.float()
    _close(y, want, dtype, scale=2.0)                                # two roundings: normalised value, then product
    # the reference's order of roundings (llada/model/modeling_llada.py:338-350); the row mean is summed in another
    # order, so a normalised value next to a rounding boundary may land on the other side (one ulp there, and the
    # product then rounds from a different value): rarely, and never more than two ulps
    two_step = (w * (s * torch.rsqrt(s.pow(2).mean(-1, keepdim=True) + 1e-5)).to(dtype)).float()
    _close(y, two_step, dtype, scale=2.0)
    if dtype != torch.float32:   # in fp32 the last bit of the scale itself depends on the summation order
        assert (y.float() == two_step).float().mean() > 0.98
    # plain norm: no delta, the first result is x itself
    same, y0 = ops.add_rms_norm(x, None, w, 1e-5)
    assert same is x
    xf = x.float()
    _close(y0, xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5) * w.float(), dtype, scale=2.0)


def test_add_rms_norm_argument_errors(device):
    x = torch.zeros(2, 8200, device=device, dtype=torch.bfloat16)
    with pytest.raises(ValueError):                                   # row longer than the kernel keeps in registers
        ops.add_rms_norm(x, None, torch.ones(8200, device=device, dtype=torch.bfloat16), 1e-5)
    x = torch.zeros(2, 12, device=device, dtype=torch.bfloat16)
    with pytest.raises(ValueError):                                   # 24-byte rows
        ops.add_rms_norm(x, None, torch.ones(12, device=device, dtype=torch.bfloat16), 1e-5)
