"""End to end on one GPU: a small Llama-style decoder wrapped with
``fully_shard`` (bf16 compute, fp32 masters), trained with gradient clipping and
the fused flat-shard AdamW.  The loss must fall like that of the same model
trained without any sharding in plain torch (fp32 masters, bf16 compute copies),
and the two must stay close step by step."""

import copy
import math

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from yafsdp_amd import MixedPrecisionPolicy

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
VOCAB, DIM, HEADS, FFN, LAYERS, SEQ = 256, 128, 4, 352, 2, 64


class RMSNorm(nn.Module):
    def __init__(self, d):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(d))

    def forward(self, x):
        v = x.float()
        return (v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + 1e-5)).to(x.dtype) * self.weight


class Layer(nn.Module):
    def __init__(self):
        super().__init__()
        self.q, self.k, self.v, self.o = (nn.Linear(DIM, DIM, bias=False) for _ in range(4))
        self.gate, self.up = nn.Linear(DIM, FFN, bias=False), nn.Linear(DIM, FFN, bias=False)
        self.down = nn.Linear(FFN, DIM, bias=False)
        self.n1, self.n2 = RMSNorm(DIM), RMSNorm(DIM)

    def forward(self, x):
        b, s, _ = x.shape
        h = self.n1(x)
        q, k, v = (m(h).view(b, s, HEADS, DIM // HEADS).transpose(1, 2) for m in (self.q, self.k, self.v))
        a = F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2).reshape(b, s, DIM)
        x = x + self.o(a)
        h = self.n2(x)
        return x + self.down(F.silu(self.gate(h)) * self.up(h))


class Embed(nn.Module):
    def __init__(self):
        super().__init__()
        self.tok = nn.Embedding(VOCAB, DIM)

    def forward(self, ids):
        return self.tok(ids)


class Llama(nn.Module):
    def __init__(self):
        super().__init__()
        self.embed = Embed()
        self.layers = nn.ModuleList([Layer() for _ in range(LAYERS)])
        self.norm = RMSNorm(DIM)
        self.head = nn.Linear(DIM, VOCAB, bias=False)

    def forward(self, ids):
        x = self.embed(ids)
        for layer in self.layers:
            x = layer(x)
        return self.head(self.norm(x))


def _batches(n):
    g = torch.Generator().manual_seed(7)
    base = torch.randint(0, VOCAB, (8, SEQ + 1), generator=g)  # a fixed set of sequences to memorise
    return [base.to(DEV) for _ in range(n)]


def _loss(model, ids):
    logits = model(ids[:, :-1])
    return F.cross_entropy(logits.float().reshape(-1, VOCAB), ids[:, 1:].reshape(-1))


def test_sharded_llama_trains_like_the_unsharded_model():
    from yafsdp_amd import fully_shard
    from yafsdp_amd.optim import FlatAdamW, grad_clip_coef

    torch.manual_seed(3)
    model0 = Llama().to(DEV)
    steps, hp = 40, dict(lr=3e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.01)
    batches = _batches(steps)

    # plain torch: fp32 masters, a bf16 copy for compute, fp32 AdamW with clipping
    ref = copy.deepcopy(model0)
    ropt = torch.optim.AdamW(ref.parameters(), **hp)
    ref_losses = []
    for ids in batches:
        low = copy.deepcopy(ref).to(torch.bfloat16)
        loss = _loss(low, ids)
        loss.backward()
        for p, q in zip(ref.parameters(), low.parameters()):
            p.grad = q.grad.float()
        torch.nn.utils.clip_grad_norm_(ref.parameters(), 1.0)
        ropt.step()
        ropt.zero_grad(set_to_none=True)
        ref_losses.append(loss.item())

    mp = MixedPrecisionPolicy(param_dtype=torch.bfloat16)
    model = copy.deepcopy(model0)
    fully_shard(model.embed, mp_policy=mp)
    for layer in model.layers:
        fully_shard(layer, mp_policy=mp)
    fully_shard([model.norm, model.head], mp_policy=mp)
    fully_shard(model, mp_policy=mp)
    opt = FlatAdamW(model.parameters(), **hp)
    losses = []
    for ids in batches:
        loss = _loss(model, ids)
        loss.backward()
        _, coef = grad_clip_coef(model, 1.0)
        opt.step(grad_scale=coef)
        opt.zero_grad(set_to_none=True)
        losses.append(loss.item())

    print("loss first/last:", losses[0], losses[-1], "reference:", ref_losses[0], ref_losses[-1],
          "max relative gap:", max(abs(a - b) / max(abs(b), 1.0) for a, b in zip(losses, ref_losses)), flush=True)
    assert all(math.isfinite(x) for x in losses)
    assert losses[0] > 5.0 and losses[-1] < 0.5 * losses[0], (losses[0], losses[-1])
    assert abs(losses[0] - ref_losses[0]) < 1e-2
    # same arithmetic up to summation order inside GEMMs and attention: the curves stay together
    for a, b in zip(losses, ref_losses):
        assert abs(a - b) <= 0.05 * max(abs(b), 1.0), (losses, ref_losses)
