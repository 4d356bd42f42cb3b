"""The torch competitor lines of the sweeps: the reference's baselines
(baselines/lm2exp.py:4-14, baselines/lt2exp.py:4-25 there), restated."""

import torch


def torch_lm2exp(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    m = torch.clamp(torch.amax(b, dim=1, keepdim=True), -1e38, 1e38)
    return m + torch.log(torch.bmm(a, torch.exp(b - m)))


def torch_lt2exp(w: torch.Tensor, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    batch, m, n = w.shape[0], w.shape[1], a.shape[2]
    ma = torch.clamp(torch.amax(a, dim=1, keepdim=True), -1e38, 1e38)
    mb = torch.clamp(torch.amax(b, dim=1, keepdim=True), -1e38, 1e38)
    s = (torch.exp(a - ma).unsqueeze(2) * torch.exp(b - mb).unsqueeze(1)).view(batch, -1, n)
    return ma + mb + torch.log(torch.bmm(w.view(batch, m, -1), s))
