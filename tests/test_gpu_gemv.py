"""GPU check of the decode driver's matrix-vector kernel (td_gemv) against a plain PyTorch fp32
reference of the same operation, with the roundings a Hugging Face Llama layer performs: the
normalised vector and silu(gate) are rounded to the storage type before they are multiplied.
Tolerance: the fp32 reference rounded to the storage type, within 2 units of that type's
precision relative to the magnitude of the accumulated terms."""
import pytest
import torch

pytestmark = pytest.mark.gpu

EPS_OF = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}


def _ref(w, x, norm_weight, eps, gated, residual, dtype):
    wf = w.float()
    if norm_weight is not None:
        xf = x.float()
        t = (xf * torch.rsqrt(xf.pow(2).mean() + eps)).to(dtype)
        f = (norm_weight * t).float()
    elif gated:
        c = w.shape[1]
        g, u = x[:c].float(), x[c:]
        f = (torch.nn.functional.silu(g).to(dtype) * u).float()
    else:
        f = x.float()
    y = wf @ f
    scale = (wf.abs() @ f.abs())
    if residual is not None:
        y = y + residual.float()
        scale = scale + residual.float().abs()
    return y, scale


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,cols,mode", [(4096, 4096, "plain"), (12288, 4096, "norm"),
                                            (4096, 11008, "gated"), (22016, 4096, "norm"),
                                            (37, 4096, "plain"), (5, 8, "plain"), (129, 16384, "gated"), (64, 28672, "plain"), (32, 30720, "norm"),
                                            (32000, 4096, "norm"), (1000, 2056, "norm")])
@pytest.mark.parametrize("with_residual", [False, True])
def test_gemv_matches_fp32_reference(cuda, dtype, rows, cols, mode, with_residual):
    from tidaldecode_amd import _kernels

    g = torch.Generator(device=cuda).manual_seed(rows * 31 + cols)
    w = (torch.randn((rows, cols), generator=g, device=cuda) * 0.05).to(dtype)
    n_x = 2 * cols if mode == "gated" else cols
    x = torch.randn(n_x, generator=g, device=cuda).to(dtype)
    nw = (1 + 0.1 * torch.randn(cols, generator=g, device=cuda)).to(dtype) if mode == "norm" else None
    res = torch.randn(rows, generator=g, device=cuda).to(dtype) if with_residual else None
    out = res.clone() if with_residual else None       # residual aliasing the output
    y = _kernels.gemv(w, x, norm_weight=nw, eps=1e-5, gated=mode == "gated",
                      residual=out, out=out)
    torch.cuda.synchronize()
    want, scale = _ref(w, x, nw, 1e-5, mode == "gated", res, dtype)
    err = (y.float() - want).abs()
    # rounding of the result to the storage type + fp32 summation order
    bound = EPS_OF[dtype] * want.abs() + 1e-5 * scale + 1e-6
    assert (err <= bound).all(), float((err / bound).max())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,cols", [(22016, 4096), (28672, 4096), (6, 64)])
def test_gemv_gate_up_pairs(cuda, dtype, rows, cols):
    """stacked gate/up projection with the activation in the epilogue == the two-launch form"""
    from tidaldecode_amd import _kernels

    g = torch.Generator(device=cuda).manual_seed(rows + cols)
    w = (torch.randn((rows, cols), generator=g, device=cuda) * 0.05).to(dtype)
    x = torch.randn(cols, generator=g, device=cuda).to(dtype)
    nw = (1 + 0.1 * torch.randn(cols, generator=g, device=cuda)).to(dtype)
    act = _kernels.gemv(w, x, norm_weight=nw, eps=1e-5, pair_gated=True)
    gu = _kernels.gemv(w, x, norm_weight=nw, eps=1e-5)          # [gate | up], rounded
    torch.cuda.synchronize()
    assert act.shape == (rows // 2,)
    want = (torch.nn.functional.silu(gu[: rows // 2].float()).to(dtype) * gu[rows // 2:])
    # same roundings; the fast exponential may flip the last bit of silu
    assert ((act.float() - want.float()).abs() <= 2 * EPS_OF[dtype] * want.float().abs() + 1e-6).all()


def test_gemv_on_a_row_slice_of_a_fused_weight(cuda):
    """rows of a larger matrix (a q/k/v block of a fused projection): the row stride is honoured"""
    from tidaldecode_amd import _kernels

    g = torch.Generator(device=cuda).manual_seed(3)
    big = (torch.randn((64, 512), generator=g, device=cuda) * 0.1).to(torch.bfloat16)
    x = torch.randn(256, generator=g, device=cuda).to(torch.bfloat16)
    w = big[8:40, :256]
    y = _kernels.gemv(w, x)
    want = w.float() @ x.float()
    assert (y.float() - want).abs().max() <= 2.0 ** -7 * want.abs().max() + 1e-4


def test_gemv_errors(cuda):
    from tidaldecode_amd import _kernels

    w = torch.zeros((16, 24), dtype=torch.bfloat16, device=cuda)
    with pytest.raises(RuntimeError):
        _kernels.gemv(w, torch.zeros(23, dtype=torch.bfloat16, device=cuda))
    with pytest.raises(RuntimeError):
        _kernels.gemv(w[:, :20], torch.zeros(20, dtype=torch.bfloat16, device=cuda))  # cols % 8
    with pytest.raises(RuntimeError):
        _kernels.gemv(w, torch.zeros(24, dtype=torch.float16, device=cuda))
    with pytest.raises(RuntimeError):
        _kernels.gemv(torch.zeros((4, 32768), dtype=torch.bfloat16, device=cuda),
                      torch.zeros(32768, dtype=torch.bfloat16, device=cuda))    # cols > 30720
