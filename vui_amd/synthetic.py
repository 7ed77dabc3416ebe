"""Random-init checkpoints of a given architecture (there is no trained checkpoint offline): the
state-dict keys and shapes of the reference model (src/vui/model.py:1076-1136, 577-663) filled
with per-key seeded N(0, std) values, norm weights 1, eos bias 0.  Used by the benchmark."""
from __future__ import annotations

import torch
from torch import Tensor

from .config import Config, DataConfig, VuiConfig, nano_config


def state_dict_shapes(m: VuiConfig) -> dict[str, tuple[int, ...]]:
    H, KV, hd, d = m.n_heads, m.kv_heads, m.head_dim, m.d_model
    sh: dict[str, tuple[int, ...]] = {}
    sh["token_emb.weight"] = (m.vocab_size, d)
    sh["audio_emb.embedding.weight"] = (m.n_quantizers * m.codebook_size, d)
    sh["codec_head.weight"] = (m.codebook_size, d)
    sh["eos_head.weight"] = (1, d)
    sh["eos_head.bias"] = (1,)
    for i in range(m.n_layers):
        p = f"decoder.blocks.{i}."
        sh[p + "attn_norm.weight"] = (d,)
        sh[p + "attn.Wqkv.weight"] = ((H + 2 * KV) * hd, d)
        sh[p + "attn.out_proj.weight"] = (d, d)
        sh[p + "mlp_norm.weight"] = (d,)
        sh[p + "mlp.w1.weight"] = (m.ffn, d)
        sh[p + "mlp.w3.weight"] = (m.ffn, d)
        sh[p + "mlp.w2.weight"] = (d, m.ffn)
    sh["decoder.norm.weight"] = (d,)
    R = m.rq_d_model
    if R != d:
        sh["rq_transformer.backbone_proj.weight"] = (R, d)
    sh["rq_transformer.code_emb.embedding.weight"] = ((m.n_quantizers - 1) * m.codebook_size, R)
    sh["rq_transformer.pos_emb.weight"] = (m.n_quantizers, R)
    sh["rq_transformer.head_W"] = (m.n_quantizers - 1, m.codebook_size, R)
    sh["rq_transformer.norm.weight"] = (R,)
    for i in range(m.rq_n_layers):
        p = f"rq_transformer.blocks.{i}."
        sh[p + "attn_norm.weight"] = (R,)
        sh[p + "Wqkv.weight"] = (3 * R, R)
        sh[p + "out_proj.weight"] = (R, R)
        sh[p + "mlp_norm.weight"] = (R,)
        sh[p + "w1.weight"] = (m.rq_ffn, R)
        sh[p + "w3.weight"] = (m.rq_ffn, R)
        sh[p + "w2.weight"] = (R, m.rq_ffn)
    return sh


def synthetic_state_dict(m: VuiConfig, seed: int = 0, std: float = 0.02) -> dict[str, Tensor]:
    """Each key draws from its own CPU generator seeded with (seed, key index)."""
    sd = {}
    for idx, (k, shape) in enumerate(state_dict_shapes(m).items()):
        g = torch.Generator().manual_seed(seed * 1000003 + idx)
        if k.endswith("norm.weight"):
            sd[k] = torch.ones(shape)
        elif k.endswith(".bias"):
            sd[k] = torch.zeros(shape)
        else:
            sd[k] = std * torch.randn(shape, generator=g)
    return sd


def nano_for_cache(preset: str, max_seqlen: int) -> Config:
    """Vui Nano with the backbone's position table / cache cut to max_seqlen positions
    (decoder.max_seqlen = max_text_tokens + max_audio_tokens + Q when data.max_secs gives 0,
    src/vui/model.py:1069-1073, 1127)."""
    cfg = nano_config(preset)
    cfg.data = DataConfig(max_secs=0)
    cfg.model.has_spk_proj = False
    cfg.model.max_text_tokens = max_seqlen - cfg.model.n_quantizers
    cfg.model.max_audio_tokens = 0
    return cfg


def synthetic_codec_state_dict(cfg, seed: int = 0) -> dict[str, Tensor]:
    """Deterministic fp32 vocoder weights (vui_amd.codec.CodecConfig) that keep activations O(1) through
    its ~60 layers: linear and conv weights N(0, 1/fan_in), biases N(0, 0.05), norm weights 1 + N(0, 0.1),
    snake log-rates N(0, 0.3), residual scales N(0.3, 0.1), codebooks N(0, 1); the closing 1x1 conv of every
    residual unit is scaled by 0.3 and the last conv by 0.12.  Each key draws from its own CPU generator
    seeded with (seed, key index)."""
    import math

    from .codec import codec_state_dict_shapes

    sd = {}
    for idx, (k, shape) in enumerate(codec_state_dict_shapes(cfg).items()):
        g = torch.Generator().manual_seed(seed * 1000003 + 7919 + idx)
        r = torch.randn(shape, generator=g)
        if k.endswith("embed"):
            t = r
        elif k.endswith(("alpha", "beta")):
            t = 0.3 * r
        elif k.endswith(("attn_scale", "mlp_scale", "gamma")):
            t = 0.3 + 0.1 * r
        elif k.endswith("norm.weight"):
            t = 1.0 + 0.1 * r
        elif k.endswith(".bias"):
            t = 0.05 * r
        elif len(shape) == 3 and (".block.1." in k or (k.startswith("upsample") and ".0.conv" in k)):
            stride = shape[2] if k.startswith("upsample") else shape[2] // 2
            t = r / math.sqrt(shape[0] * shape[2] / stride)
        elif len(shape) == 3:
            t = r / math.sqrt(shape[1] * shape[2])
            if "conv2.conv" in k:
                t = 0.3 * t
            elif shape[0] == 1:
                t = 0.12 * t
        else:
            t = r / math.sqrt(shape[-1])
        sd[k] = t.contiguous()
    return sd
