"""The path on CPU tensors with stock PyTorch, timed by bench.py as the reported CPU
baseline (``cpu_baseline.kind = "port"``).  TEST / MEASUREMENT INFRASTRUCTURE ONLY.

The reference has no CPU path (llama3_inference.py:18 asserts a GPU; RMSNorm and rotary
embedding exist only as kernels, model.py:71,100-101), so this is a restatement of the same
math with the routines the reference itself compares against or calls:
  * attention: F.scaled_dot_product_attention(q, k, v, enable_gqa=True) on the same strided
    bf16 views (benchmark_kernel.py:27-28, model.py:116);
  * RMSNorm: the formula of custom_kernels.cu:343-344 in float32, rounded once;
  * rotary: complex multiply by the table rows (custom_kernels.cu:400-414, model.py:51-60).
"""

import torch
import torch.nn.functional as F


def attention_cpu(q, k, v):
    return F.scaled_dot_product_attention(q, k, v, enable_gqa=True)


def rms_norm_cpu(x, w, eps):
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(x.dtype)


def rot_embed_cpu(x, freq):
    B, T, NH, HD = x.shape
    xc = torch.view_as_complex(x.float().reshape(B, T, NH, HD // 2, 2))
    fc = torch.view_as_complex(freq.reshape(T, HD // 2, 2))
    return torch.view_as_real(xc * fc[None, :, None, :]).flatten(3).to(x.dtype)
