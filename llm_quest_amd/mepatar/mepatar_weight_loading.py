"""Checkpoint import of Mepatar: ``config.json`` + ``model.safetensors`` of a model folder -> ``MepatarModel``.

Tensor names of the checkpoint: ``embed``, ``head``, ``final.norm``, and per layer i ``l<i>.norm1|norm2``, ``l<i>.canon1`` (the input convolution),
``l<i>.mix.*`` (retention: q, k, v, g, o; attention: q, k, v, o each with ``.b``, q.norm, k.norm, temp; delta: q, k, v each with ``.conv``, b, a, A_log,
dt_bias, norm, g, o) and ``l<i>.mlp.*`` (dense: gate, up, down; experts: router, e<j>.gate, e<j>.up, e<j>.down).  Projections that share their input are
stored side by side in one parameter, the experts of a layer stacked in one (gate and up rows in alternating blocks of 32, so that the gated activation is
the product's epilogue), so that each group is one product.
"""

import json
import os

import torch

from llm_quest_amd.common.mixers import GatedDeltaRule, GatedMLP, Retention, SlidingWindowAttention
from llm_quest_amd.gemepel.gemepel_weight_loading import _put
from llm_quest_amd.mepatar.mepatar_model import MepatarConfig, MepatarModel


def load_mepatar(model_dir, act_dtype=torch.bfloat16, device="cuda"):
    from safetensors.torch import load_file

    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = MepatarConfig(json.load(f))
    model = MepatarModel(cfg, act_dtype=act_dtype)
    load_mepatar_state(model, load_file(os.path.join(model_dir, "model.safetensors")))
    return model.to(device)


def load_mepatar_state(model, w):
    """Copy the checkpoint tensors ``w`` (name -> tensor) into the model's fused parameters."""
    _put(model.embed, w["embed"])
    _put(model.head, w["head"])
    _put(model.final_norm, w["final.norm"])
    for i, blk in enumerate(model.blocks):
        p, mx = f"l{i}.", blk.mixer
        _put(blk.norm1, w[p + "norm1"])
        _put(blk.canon.weight, w[p + "canon1"])
        m = p + "mix."
        if isinstance(mx, Retention):
            _put(mx.w_in, w[m + "q"], w[m + "k"], w[m + "v"], w[m + "g"])
        elif isinstance(mx, SlidingWindowAttention):
            _put(mx.w_qkv, w[m + "q"], w[m + "k"], w[m + "v"])
            _put(mx.b_qkv, w[m + "q.b"], w[m + "k.b"], w[m + "v.b"])
            _put(mx.q_norm, w[m + "q.norm"])
            _put(mx.k_norm, w[m + "k.norm"])
            _put(mx.temp, w[m + "temp"])
            _put(mx.b_o, w[m + "o.b"])
        elif isinstance(mx, GatedDeltaRule):
            _put(mx.w_in, w[m + "q"], w[m + "k"], w[m + "v"], w[m + "g"], w[m + "b"], w[m + "a"])
            _put(mx.conv, w[m + "q.conv"], w[m + "k.conv"], w[m + "v.conv"])
            _put(mx.A_log, w[m + "A_log"])
            _put(mx.dt_bias, w[m + "dt_bias"])
            _put(mx.norm, w[m + "norm"])
        _put(mx.w_o, w[m + "o"])
        if blk.ff is None:
            continue
        _put(blk.norm2, w[p + "norm2"])
        e = p + "mlp."
        if isinstance(blk.ff, GatedMLP):
            _put(blk.ff.w_gate_up, w[e + "gate"], w[e + "up"])
            _put(blk.ff.w_down, w[e + "down"])
        else:
            _put(blk.ff.w_router, w[e + "router"])
            n = range(blk.ff.experts)
            blk.ff.load_experts([w[f"{e}e{j}.gate"] for j in n], [w[f"{e}e{j}.up"] for j in n], [w[f"{e}e{j}.down"] for j in n])
    return model
