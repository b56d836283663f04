"""Residual add fused with LayerNorm (HIP kernel s3d_add_layernorm) for the Swin block around the
attention operator (Swin3D/modules/swin3d_layers.py:617-623)."""
import torch

from . import _lib

_DTYPE_CODE = {torch.float32: _lib.S3D_DTYPE_F32, torch.float16: _lib.S3D_DTYPE_F16}


def add_layernorm(x, residual, norm, out_dtype=torch.float16, inplace=False):
    """(x + residual, LayerNorm(x + residual)) for x fp32 [N,C] on the GPU and `norm` a torch.nn.LayerNorm over C.

    residual   fp16 / fp32 [N,C] or None (then the first result is x itself)
    out_dtype  dtype of the normalised rows (fp16: what the next GEMM reads under autocast)
    inplace    write the sum back into x instead of a new tensor
    No autograd: for inference, or inside torch.no_grad().
    """
    if not x.is_cuda or x.dtype != torch.float32 or x.dim() != 2:
        raise ValueError(f"x must be a float32 [N,C] CUDA (HIP) tensor, got {x.dtype} {tuple(x.shape)} on {x.device}")
    n, c = x.shape
    if tuple(norm.normalized_shape) != (c,) or norm.weight is None or norm.bias is None:
        raise ValueError("norm must be an affine LayerNorm over the channel axis")
    if out_dtype not in _DTYPE_CODE:
        raise ValueError(f"out_dtype {out_dtype} (float16 or float32)")
    x = x.contiguous()
    res_ptr, res_code = None, 0
    summed = x
    if residual is not None:
        if residual.shape != x.shape or residual.dtype not in _DTYPE_CODE or residual.device != x.device:
            raise ValueError("residual must be float16/float32 of x's shape on x's device")
        residual = residual.contiguous()
        res_ptr, res_code = residual.data_ptr(), _DTYPE_CODE[residual.dtype]
        summed = x if inplace else torch.empty_like(x)
    y = torch.empty((n, c), dtype=out_dtype, device=x.device)
    gamma, beta = norm.weight.detach().float().contiguous(), norm.bias.detach().float().contiguous()
    with torch.cuda.device(x.device):
        stream = torch.cuda.current_stream(x.device).cuda_stream
        status = _lib.lib().s3d_add_layernorm(x.data_ptr(), res_ptr, res_code, gamma.data_ptr(), beta.data_ptr(),
                                             float(norm.eps), summed.data_ptr() if residual is not None else None,
                                             y.data_ptr(), _DTYPE_CODE[out_dtype], n, c, stream)
    _lib.check(status, "s3d_add_layernorm")
    return summed, y
