"""AdamW oracle (CPU, fp32).  Test infrastructure — see oracle/__init__.py.

Restates flextrain/ops/_kernels/adamw.py:34-56 and the host-side bias
corrections of :73-75: decay, moments, bias-corrected step, all fp32, results
stored back in each buffer's dtype.
"""
from __future__ import annotations

import torch


def adamw_step(p, g, m, v, lr=1e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.001, step=1):
    """Returns new (p, m, v) in their input dtypes plus bf16(p_new)."""
    step = max(1, step)
    bc1 = torch.tensor(1.0 - beta1 ** step, dtype=torch.float32)
    bc2 = torch.tensor(1.0 - beta2 ** step, dtype=torch.float32)
    f = lambda s: torch.tensor(s, dtype=torch.float32)
    pf, gf, mf, vf = p.float(), g.float(), m.float(), v.float()
    pf = pf - (f(lr) * f(weight_decay)) * pf
    mf = f(beta1) * mf + (1.0 - f(beta1)) * gf
    vf = f(beta2) * vf + (1.0 - f(beta2)) * (gf * gf)
    pf = pf - f(lr) * ((mf / bc1) / (torch.sqrt(vf / bc2) + f(eps)))
    return pf.to(p.dtype), mf.to(m.dtype), vf.to(v.dtype), pf.to(torch.bfloat16)
