"""The scans inside a small linear-RNN layer, the way their callers use them
(README.md:8,42 of the reference: gates and tokens come out of projections, the
states go into one): parameter gradients through the HIP operators against the
same layer evaluated with a plain time loop in fp64 on the CPU, for every scan
flavour of the package, and a few optimiser steps that must lower the loss.
"""

import pytest
import torch

pytestmark = pytest.mark.gpu

DEVICE = "cuda"


def _loop(gates, tokens, reverse=False):
    """x[t] = gates[t] x[t-1] + tokens[t] as a Python loop over (B, C, T) tensors (autograd-friendly)."""
    T = gates.shape[-1]
    order = range(T - 1, -1, -1) if reverse else range(T)
    state = torch.zeros_like(gates[..., 0])
    out = [None] * T
    for t in order:
        state = gates[..., t] * state + tokens[..., t]
        out[t] = state
    return torch.stack(out, dim=-1)


class Layer(torch.nn.Module):
    """y = W_o scan(gate(W_g u), W_x u): `mix` says how the gate and the token are formed."""

    def __init__(self, dim, hidden, mix, device, dtype):
        super().__init__()
        gen = torch.Generator().manual_seed(11)
        mk = lambda *s: torch.nn.Parameter((torch.randn(*s, generator=gen) / s[-1] ** 0.5).to(device=device, dtype=dtype))
        self.w_gate, self.w_token, self.w_out = mk(hidden, dim), mk(hidden, dim), mk(dim, hidden)
        self.mix = mix

    def forward(self, u, fused):
        # u: (B, T, dim) -> channels first, time last, contiguous, as the scans want it
        z = torch.einsum("hd,btd->bht", self.w_gate, u).contiguous()
        v = torch.einsum("hd,btd->bht", self.w_token, u).contiguous()
        if fused:
            from accelerated_scan import complex as cscan
            from accelerated_scan import gated, ref, scalar, warp

            if self.mix == "sigmoid":
                x = gated.sigmoid_scan(z, v)
            elif self.mix == "lerp":
                x = gated.sigmoid_lerp_scan(z, v)
            elif self.mix == "exp_norm":
                x = gated.exp_norm_scan(-torch.nn.functional.softplus(z) - 1e-3, v)
            elif self.mix == "bidirectional":
                a = torch.sigmoid(z)
                x = warp.scan(a, v) + ref.scan(a, v, reverse=True)
            elif self.mix == "scalar":
                x = scalar.scan(torch.sigmoid(z), v)
            else:  # complex gates of modulus sigmoid(z) and phase v, real tokens
                x = cscan.scan(torch.polar(torch.sigmoid(z), v), v).real
        else:
            if self.mix == "sigmoid" or self.mix == "scalar":
                x = _loop(torch.sigmoid(z), v)
            elif self.mix == "lerp":
                a = torch.sigmoid(z)
                x = _loop(a, (1 - a) * v)
            elif self.mix == "exp_norm":
                logs = -torch.nn.functional.softplus(z) - 1e-3
                x = _loop(torch.exp(logs), torch.sqrt(-torch.expm1(2 * logs)) * v)
            elif self.mix == "bidirectional":
                a = torch.sigmoid(z)
                x = _loop(a, v) + _loop(a, v, reverse=True)
            else:
                x = _loop(torch.polar(torch.sigmoid(z), v), v.to(torch.complex128)).real
        return torch.einsum("dh,bht->btd", self.w_out, x)


MIXES = ["sigmoid", "lerp", "exp_norm", "bidirectional", "scalar", "complex"]


@pytest.mark.parametrize("mix", MIXES)
def test_parameter_gradients_match_the_time_loop(mix):
    B, T, dim, hidden = 2, 300, 24, 40
    gen = torch.Generator().manual_seed(3)
    u = torch.randn(B, T, dim, generator=gen)
    target = torch.randn(B, T, dim, generator=gen)

    fused = Layer(dim, hidden, mix, DEVICE, torch.float32)
    loss = (fused(u.to(DEVICE), fused=True) - target.to(DEVICE)).square().mean()
    loss.backward()

    plain = Layer(dim, hidden, mix, "cpu", torch.float64)
    loss_ref = (plain(u.double(), fused=False) - target.double()).square().mean()
    loss_ref.backward()

    assert abs(loss.item() - loss_ref.item()) <= 1e-5 * abs(loss_ref.item())
    for (name, p), (_, q) in zip(fused.named_parameters(), plain.named_parameters()):
        scale = q.grad.abs().max().item()
        torch.testing.assert_close(p.grad.cpu().double(), q.grad, rtol=2e-4, atol=2e-5 * scale,
                                   msg=lambda m: f"{mix} {name}: {m}")


@pytest.mark.parametrize("mix", ["lerp", "exp_norm"])
def test_a_few_optimiser_steps_lower_the_loss(mix):
    B, T, dim, hidden = 4, 2048, 32, 64
    gen = torch.Generator().manual_seed(5)
    u = torch.randn(B, T, dim, generator=gen).to(DEVICE)
    # the target is a moving average of the input: something a gated scan can fit
    target = torch.nn.functional.avg_pool1d(u.transpose(1, 2), 9, stride=1, padding=4, count_include_pad=True).transpose(1, 2)
    layer = Layer(dim, hidden, mix, DEVICE, torch.float32)
    opt = torch.optim.Adam(layer.parameters(), lr=3e-2)
    losses = []
    for _ in range(30):
        opt.zero_grad()
        loss = (layer(u, fused=True) - target).square().mean()
        loss.backward()
        opt.step()
        losses.append(loss.item())
    assert all(l == l for l in losses)  # no NaN
    assert losses[-1] < 0.6 * losses[0], losses
