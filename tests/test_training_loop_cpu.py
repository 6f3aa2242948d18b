"""A few optimizer steps of a small two-layer transformer built on the dense operator, on the task of the
reference's example (example/test_transformer.py:33-68: among random tokens two carry the same symbol; predict the
distance between their position codes), once with l1attn_cpp.L1Attn and once with the same graph on torch's own
autograd through the closed form for the logits.  Same initial weights, same batches, float64: the weights after
the steps must agree to rounding, which they only do if every gradient the operator hands back is right in a
loop where its inputs are themselves functions of trained weights.  The GPU operator runs the same loop in the
GPU tests."""
import torch
from torch import nn

import closed_forms as cf
import model_blocks as mb


def make_batch(g, batch, n_ctx, n_symb):
    x = torch.zeros(batch, n_ctx, n_symb + 2, dtype=torch.float64)
    x[:, :, :n_symb] = torch.randn(batch, n_ctx, n_symb, generator=g, dtype=torch.float64) / 2
    i = torch.randint(n_ctx, (batch,), generator=g)
    j = torch.remainder(i + torch.randint(n_ctx - 1, (batch,), generator=g) + 1, n_ctx)
    r = torch.arange(batch)
    x[r, i, :n_symb] = x[r, j, :n_symb]                       # the matching pair
    x[:, :, -2] = torch.randint(128, (batch, n_ctx), generator=g).double() / 16.0   # position code
    x[:, :, -1] = x[:, :, -2] / 4
    return x, (x[r, i, -2] - x[r, j, -2]).abs()


class Net(nn.Module):
    def __init__(self, indim, width, n_head, n_layers, l1a, seed):
        super().__init__()
        g = torch.Generator().manual_seed(seed)
        mk = lambda *s: nn.Parameter(torch.randn(*s, generator=g, dtype=torch.float64) / s[0] ** 0.5)
        self.enc, self.dec = mk(indim, width), mk(width, 1)
        self.w = nn.ParameterList([mk(width, 3 * width) for _ in range(n_layers)])
        self.b = nn.ParameterList([nn.Parameter(torch.zeros(3 * width, dtype=torch.float64)) for _ in range(n_layers)])
        self.n_head, self.l1a = n_head, l1a

    def forward(self, x):
        x = torch.tanh(x @ self.enc)
        for w, b in zip(self.w, self.b):
            x = mb.split_block(x, w, b, self.l1a, self.n_head)
        return (x @ self.dec)[:, :, 0].sum(1)


def train(l1a, steps=6):
    net = Net(indim=8, width=24, n_head=2, n_layers=2, l1a=l1a, seed=3)
    opt = torch.optim.Adam(net.parameters(), lr=2e-3)
    g = torch.Generator().manual_seed(11)
    losses = []
    for _ in range(steps):
        x, y = make_batch(g, batch=16, n_ctx=12, n_symb=6)
        loss = ((net(x) - y) ** 2).mean()
        opt.zero_grad()
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    return net, losses


def test_training_steps_match_torch_autograd():
    import l1attn_cpp
    net_a, loss_a = train(l1attn_cpp.L1Attn())
    net_b, loss_b = train(cf.dense_attn)
    for la, lb in zip(loss_a, loss_b):
        assert abs(la - lb) <= 1e-9 * max(1.0, abs(lb))
    for pa, pb in zip(net_a.parameters(), net_b.parameters()):
        assert cf.rel_err(pa.detach(), pb.detach()) <= 1e-9
    assert all(torch.isfinite(p).all() for p in net_a.parameters())
