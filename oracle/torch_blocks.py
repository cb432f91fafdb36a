"""Stock-PyTorch CPU restatement of the reference MoE blocks -- TEST INFRASTRUCTURE.

Two uses only: (1) the ``cpu_baseline`` leg of ``bench.py`` times it on the host
cores, (2) tests use it as a second witness for the C oracle (it relies on
torch's own softmax/sigmoid/topk/argsort/linear, so it shares no arithmetic with
``moe_oracle.c``).  It keeps the reference's structure -- fp32 gate, a Python
loop over experts, bf16 ``F.linear`` per expert in chunks of at most
``chunk`` rows, fp8 block dequantisation per expert call -- but uses
``sorted=True`` / ``stable=True`` so that its index outputs are comparable with
the canonical ones wherever the scores have no ties.

Follows: modeling_deepseek_v3.py:439-711, modeling_deepseek_v2.py:425-566 and
:662-758, Wrapper.py:109-138 and :470-530; Mixtral per transformers 4.42.0
(MixtralSparseMoeBlock / MixtralBlockSparseTop2MLP), which the reference imports
but does not vendor.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F


def dequant(q_fp8: torch.Tensor, scale: torch.Tensor, block: int = 128) -> torch.Tensor:
    """Wrapper.py:109-138."""
    rows, cols = q_fp8.shape
    s = scale.repeat_interleave(block, 0).repeat_interleave(block, 1)[:rows, :cols]
    return (q_fp8.to(torch.float32) * s).to(torch.bfloat16)


def quant(x: torch.Tensor, block: int = 128):
    """deepseekv3_initializer.py:191-205 (per 128x128 block amax scaling)."""
    m, n = x.shape
    mp, np_ = math.ceil(m / block) * block, math.ceil(n / block) * block
    xp = torch.zeros(mp, np_, dtype=x.dtype)
    xp[:m, :n] = x
    v = xp.view(mp // block, block, np_ // block, block)
    amax = v.abs().float().amax(dim=(1, 3), keepdim=True).clamp(1e-4)
    q = (v * (448.0 / amax)).to(torch.float8_e4m3fn).view(mp, np_)[:m, :n].contiguous()
    return q, (amax / 448.0).view(mp // block, np_ // block)


def _group_mask(group_scores, topk_group, per):
    gi = torch.topk(group_scores, k=topk_group, dim=-1, sorted=True)[1]
    gm = torch.zeros_like(group_scores)
    gm.scatter_(1, gi, 1)
    return gm.unsqueeze(-1).expand(-1, -1, per).reshape(group_scores.shape[0], -1).bool()


def gate_v3(x2d, weight, bias, top_k, n_group, topk_group, norm_topk_prob, scale):
    """modeling_deepseek_v3.py:500-561 (sigmoid + e_score_correction_bias, noaux_tc)."""
    n = x2d.shape[0]
    logits = F.linear(x2d.float(), weight.float())
    scores = logits.sigmoid()
    choice = scores + bias.unsqueeze(0)
    E = scores.shape[1]
    gs = choice.view(n, n_group, -1).topk(2, dim=-1)[0].sum(dim=-1)
    mask = _group_mask(gs, topk_group, E // n_group)
    tmp = choice.masked_fill(~mask, 0.0)
    idx = torch.topk(tmp, k=top_k, dim=-1, sorted=True)[1]
    w = scores.gather(1, idx)
    if top_k > 1 and norm_topk_prob:
        w = w / (w.sum(dim=-1, keepdim=True) + 1e-20)
    return idx, w * scale, logits


def gate_v2(x2d, weight, top_k, method, n_group, topk_group, norm_topk_prob, scale):
    """modeling_deepseek_v2.py:483-533 (softmax; greedy or group_limited_greedy)."""
    n = x2d.shape[0]
    logits = F.linear(x2d.float(), weight.float())
    scores = logits.softmax(dim=-1, dtype=torch.float32)
    if method == "greedy":
        w, idx = torch.topk(scores, k=top_k, dim=-1, sorted=True)
    elif method == "group_limited_greedy":
        gs = scores.view(n, n_group, -1).max(dim=-1).values
        mask = _group_mask(gs, topk_group, scores.shape[1] // n_group)
        w, idx = torch.topk(scores.masked_fill(~mask, 0.0), k=top_k, dim=-1, sorted=True)
    else:
        raise NotImplementedError(method)
    if top_k > 1 and norm_topk_prob:
        w = w / (w.sum(dim=-1, keepdim=True) + 1e-20)
    else:
        w = w * scale
    return idx, w, logits


def gate_mixtral(x2d, weight, top_k=2):
    """bf16 gate Linear, fp32 softmax, top-k, renormalise, cast to bf16."""
    logits = F.linear(x2d, weight)  # bf16
    p = F.softmax(logits, dim=1, dtype=torch.float)
    w, idx = torch.topk(p, top_k, dim=-1)
    w = w / w.sum(dim=-1, keepdim=True)
    return idx, w.to(x2d.dtype), logits


def swiglu(x, wg, wu, wd):
    """down(silu(gate(x)) * up(x)) with bf16 Linear layers."""
    return F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd)


def expert_call(x, weights, chunk):
    """Expert_Wrapper.forward (Wrapper.py:470-530): fetch (and, for fp8, dequantise)
    the three matrices, then run the MLP in chunks of at most `chunk` rows."""
    mats = []
    for wq in weights:
        mats.append(dequant(*wq) if isinstance(wq, tuple) else wq)
    out = torch.zeros_like(x)
    for s in range(0, x.shape[0], chunk):
        out[s:s + chunk] = swiglu(x[s:s + chunk], *mats)
    return out


def moe_infer(x, idx, w, experts, chunk, v2_bf16_weights):
    """modeling_deepseek_v3.py:629-711 / modeling_deepseek_v2.py:671-758, ep_size == 1."""
    n, k = idx.shape
    E = len(experts)
    cnts = idx.new_zeros((n, E))
    cnts.scatter_(1, idx, 1)
    per_expert = cnts.sum(dim=0).tolist()
    order = idx.view(-1).argsort(stable=True)
    sorted_tokens = x[order // k]
    outs, start = [], 0
    for e, m in enumerate(per_expert):
        if m == 0:
            continue
        outs.append(expert_call(sorted_tokens[start:start + m], experts[e], chunk))
        start += m
    outs = torch.cat(outs, dim=0) if outs else sorted_tokens.new_empty(0)
    new_x = torch.empty_like(outs)
    new_x[order] = outs
    if v2_bf16_weights:
        w = w.to(new_x.dtype)
    return (new_x.view(n, k, -1).type(w.dtype).mul_(w.unsqueeze(-1)).sum(dim=1).type(new_x.dtype))


@torch.no_grad()
def deepseek_block(x, gate_w, bias, experts, shared, family, top_k, method="greedy",
                   n_group=1, topk_group=1, norm_topk_prob=False, scale=1.0, chunk=2048):
    """DeepseekV3MoE.forward (:614-626) / DeepseekV2MoE.forward (:642-668), inference."""
    shape = x.shape
    x2d = x.view(-1, shape[-1])
    if family == "v3":
        idx, w, _ = gate_v3(x2d, gate_w, bias, top_k, n_group, topk_group, norm_topk_prob, scale)
    else:
        idx, w, _ = gate_v2(x2d, gate_w, top_k, method, n_group, topk_group, norm_topk_prob, scale)
    y = moe_infer(x2d, idx, w, experts, chunk, family == "v2").view(*shape)
    if shared is not None:
        y = y + expert_call(x2d, shared, chunk).view(*shape)
    return y


@torch.no_grad()
def mixtral_block(x, gate_w, experts, top_k=2, chunk=2048):
    """MixtralSparseMoeBlock.forward of transformers 4.42.0: per expert in index
    order, index_add_ of the weighted expert output into a bf16 accumulator."""
    shape = x.shape
    x2d = x.view(-1, shape[-1])
    idx, w, logits = gate_mixtral(x2d, gate_w, top_k)
    out = torch.zeros_like(x2d)
    mask = F.one_hot(idx, num_classes=len(experts)).permute(2, 1, 0)
    for e in range(len(experts)):
        slot, tok = torch.where(mask[e])
        if tok.numel() == 0:
            continue
        cur = expert_call(x2d[tok], experts[e], chunk) * w[tok, slot, None]
        out.index_add_(0, tok, cur.to(x2d.dtype))
    return out.view(*shape), logits
