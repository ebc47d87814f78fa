"""Sequence mixers of the hybrid (layer-list) model family, one function per kind.

Every mixer maps the normed layer input ``h`` [T, D] (storage dtype) to the layer's update
[T, D] in fp32, reading and writing its run's cache or state. They share one calling form so a
design lists its layers by kind (``MIXERS``):

    y = MIXERS[spec.kind](spec, lp, h, step, cache, eps)

``lp``: the layer's tensors (``models/weights.hybrid_layer_shapes``) plus the constants
derived at load time (``derive_constants``); ``step``: the per-step metadata (``StepView``);
``cache``: this run's entry of ``engine.kv_cache.HybridCache``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from ..ops import hybrid as H
from .configs import LayerSpec


@dataclass
class StepView:
    """What the mixers need of a step: packed tokens of S sequences, each a run of consecutive
    rows [cu[s], cu[s+1]) at consecutive positions, attending through its block table."""
    cu_seqlens: torch.Tensor        # [S+1] int32
    max_seqlen: int
    positions: torch.Tensor         # [T] int32
    slot_mapping: torch.Tensor      # [T] int32, cache row of each token (-1: not stored)
    block_tables: torch.Tensor      # [S, W] int32
    block_size: int
    state_slots: Optional[torch.Tensor]   # [S] int32 recurrent-state slot (-1: padding row)


def derive_constants(spec: LayerSpec, lp: dict, device) -> None:
    """Constants a design fixes by formula, computed once (float64 on the host, stored fp32)."""
    if spec.kind == "attention":
        # per-head slope of the linear distance bias: 2^(-8 (h+1) / H)
        h = torch.arange(1, spec.heads + 1, dtype=torch.float64)
        lp["slopes"] = torch.pow(2.0, -8.0 * h / spec.heads).float().to(device)
        lp["talk"] = lp["talk"].float().contiguous()
    elif spec.kind == "latent_attention":
        i = torch.arange(spec.rot_dims // 2, dtype=torch.float64)
        lp["inv_freq"] = torch.pow(spec.rot_base, -2.0 * i / max(1, spec.rot_dims)).float().to(device)
    elif spec.kind == "talk_attention":
        lp["talk"] = lp["talk"].float().contiguous()
    if spec.ff_kind == "moe" and spec.ff:
        lp["correction"] = lp["correction"].float().contiguous()


def attention_mixer(spec: LayerSpec, lp: dict, h, step: StepView, cache, eps: float):
    """Windowed softmax attention: per-head RMS-normed q / k, values = the un-normed keys,
    linear distance bias, the heads' softmax weights mixed by ``talk``, sigmoid output gate."""
    Hh, G, d = spec.heads, spec.kv_heads, spec.dim
    kc, vc = cache
    proj = H.linear_any(h, lp["w_in"])                       # fp32 [T, q | k | gate]
    q = H.attn_prepare(proj, lp["q_norm"], lp["k_norm"], eps, Hh, G, d, kc, vc,
                       step.slot_mapping)
    gate = proj[:, (Hh + G) * d:]
    o = H.window_attention(q, kc, vc, d, d, Hh, G, step.cu_seqlens, step.max_seqlen,
                           step.positions, step.block_tables, step.block_size, spec.window,
                           spec.scale, slopes=lp["slopes"], talk=lp["talk"], gate=gate)
    return H.linear_any(o, lp["wo"])


def hgrn2_mixer(spec: LayerSpec, lp: dict, h, step: StepView, cache, eps: float):
    """Gated linear recurrence: the forget gate (bounded below by ``lower``) also sets what is
    written; per-head RMS norm of the read-out."""
    (state,) = cache
    proj = H.linear_any(h, lp["w_in"])                       # fp32 [T, q | f | v]
    o = H.hgrn2(proj, lp["f_b"], lp["lower"], lp["o_norm"], eps, state, step.state_slots,
                step.cu_seqlens, step.max_seqlen, step.positions, spec.heads, spec.dim,
                spec.vdim)
    return H.linear_any(o, lp["wo"])


def latent_attention_mixer(spec: LayerSpec, lp: dict, h, step: StepView, cache, eps: float):
    """Latent attention in the absorbed form. Only the normed latent c and the shared rotated
    key are cached. With k_h = W_uk,h c and v_h = W_uv,h c,
        q_h . k_h = (W_uk,h^T q_h) . c      and      sum_j w_j v_h,j = W_uv,h (sum_j w_j c_j),
    so every head attends the same cached row [c | k_rot] with the query [W_uk,h^T q_h | q_rot]
    and its output is expanded afterwards: one multi-query attention over the latent, for
    prompts and decoding alike, and no per-step expansion of the window's keys."""
    Hh, d, dr, dv, r = spec.heads, spec.dim, spec.rot_dim, spec.vdim, spec.kv_rank
    (c,) = cache
    T = h.shape[0]
    proj = H.linear_any(h, lp["w_in"])                       # fp32 [T, q heads | ckv | k_rot]
    q_nope, q_full = H.mla_prepare(proj, lp["c_norm"], eps, Hh, d, dr, r, spec.rot_dims,
                                   lp["inv_freq"], step.positions, step.slot_mapping, c)
    H.head_linear(q_nope, lp["w_ukT"], q_full)               # q_full[:, h, :r] = W_uk,h^T q_h
    ol = H.window_attention(q_full.view(T, Hh * (r + dr)), c, c, r + dr, r, Hh, 1,
                            step.cu_seqlens, step.max_seqlen, step.positions,
                            step.block_tables, step.block_size, spec.window, spec.scale)
    o = torch.empty(T, Hh, dv, dtype=h.dtype, device=h.device)
    H.head_linear(ol.view(T, Hh, r), lp["w_uv"], o)
    return H.linear_any(o.view(T, Hh * dv), lp["wo"])


def talk_attention_mixer(spec: LayerSpec, lp: dict, h, step: StepView, cache, eps: float):
    """Softmax attention inside blocks of ``spec.chunk`` positions: biased q / k / v, unit-RMS
    q and k, the heads' scores mixed by ``talk`` before the softmax. The mixing is folded into
    the queries (``ops.hybrid.talk_prepare``), so the attention itself is the plain kernel with
    one key head spanning the cached row and G value heads. ``cache`` may be another layer's
    (``spec.kv_from``): then only queries are projected."""
    Hh, G, d, dv = spec.heads, spec.kv_heads, spec.dim, spec.vdim
    kc, vc = cache
    proj = H.linear_any(h, lp["w_in"])                       # fp32 [T, q (| k | v)]
    q = H.talk_prepare(proj, lp["b_in"], lp["talk"], eps, Hh, G, d, dv, kc, vc,
                       step.slot_mapping, own_kv=spec.kv_from < 0)
    o = H.window_attention(q, kc, vc, G * d, dv, Hh, G, step.cu_seqlens, step.max_seqlen,
                           step.positions, step.block_tables, step.block_size,
                           spec.window or (1 << 30), spec.scale, chunk=spec.chunk, k_groups=1)
    return H.linear_any(o, lp["wo"])


MIXERS = {"attention": attention_mixer, "hgrn2": hgrn2_mixer,
          "latent_attention": latent_attention_mixer, "talk_attention": talk_attention_mixer}


# ----------------------------------------------------------------------------- feed-forwards
def gated_gelu_ff(spec: LayerSpec, lp: dict, h):
    act = H.act_mul(H.linear_any(h, lp["w_gu"]), spec.ff, h.dtype, "gelu_mul")
    return H.linear_any(act, lp["w_down"])


def gelu_ff(spec: LayerSpec, lp: dict, h):
    act = H.act_mul(H.linear_any(h, lp["w_up"]), spec.ff, h.dtype, "gelu")
    return H.linear_any(act, lp["w_down"])


def moe_ff(spec: LayerSpec, lp: dict, h):
    """Routed gated-SiLU experts + identity experts + a gated shared expert, summed in fp32."""
    ng = 1 if spec.shared_ff else 0
    tw, ti, gates = H.score_router(h, lp["router"], lp["correction"], spec.top, ng)
    shared = (lp["ws_gu"], lp["ws_down"], gates) if ng else None
    return H.moe_experts_f32(h, lp["w_gu"], lp["w_down"], tw, ti, shared)


FEED_FORWARDS = {"gated_gelu": gated_gelu_ff, "gelu": gelu_ff, "moe": moe_ff}
