"""Producer of the (positions, head_dim) float32 cos/sin table that rot_embed consumes.

Counterpart of precompute_freqs_cis / apply_scaling (model.py:27-60).  The table layout is
the reference's: row t = [cos(t f0), sin(t f0), cos(t f1), sin(t f1), ...].  The Llama-3
wavelength banding takes its parameters as arguments (model.py:29-32 hard-codes factor 8,
low 1, high 4, context 8192; Llama-3.2 checkpoints use factor 32).
"""

import math

import torch


def apply_scaling(freqs: torch.Tensor, scale_factor: float = 8.0, low_freq_factor: float = 1.0,
                  high_freq_factor: float = 4.0, old_context_len: int = 8192) -> torch.Tensor:
    """Llama-3 frequency banding: keep short wavelengths, divide long ones by scale_factor,
    blend linearly in between (model.py:34-48), vectorised."""
    wavelen = 2 * math.pi / freqs
    low_freq_wavelen = old_context_len / low_freq_factor
    high_freq_wavelen = old_context_len / high_freq_factor
    smooth = (old_context_len / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
    blended = (1 - smooth) * freqs / scale_factor + smooth * freqs
    out = torch.where(wavelen > low_freq_wavelen, freqs / scale_factor, blended)
    out = torch.where(wavelen < high_freq_wavelen, freqs, out)
    return out.to(freqs.dtype)


def precompute_freqs_cis(dim: int, end: int, theta: float = 10000.0, use_scaled: bool = False,
                         scale_factor: float = 8.0, low_freq_factor: float = 1.0,
                         high_freq_factor: float = 4.0, old_context_len: int = 8192,
                         device=None) -> torch.Tensor:
    """(end, dim) float32 table of interleaved (cos, sin); same positional arguments as
    model.py:51-53.  Built on the CPU so the table does not depend on the device's
    pow/sincos, then moved to ``device``."""
    freqs = 1.0 / (theta ** (torch.arange(0, dim, 2, device="cpu")[: (dim // 2)].float() / dim))
    if use_scaled:
        freqs = apply_scaling(freqs, scale_factor, low_freq_factor, high_freq_factor, old_context_len)
    t = torch.arange(end, device="cpu", dtype=torch.float32)
    angle = torch.outer(t, freqs)
    table = torch.stack((torch.cos(angle), torch.sin(angle)), dim=-1).flatten(1)
    return table if device is None else table.to(device)
