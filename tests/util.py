"""Helpers shared by the tests: oracle dims <-> product config, model construction."""
import torch

from oracle import vui_oracle as O


def dims_to_config(d: O.Dims, max_seqlen: int | None = None):
    from vui_amd.config import Config, DataConfig, VuiConfig

    m = VuiConfig(d_model=d.d_model, n_layers=d.n_layers, n_heads=d.n_heads, n_kv_heads=d.n_kv_heads,
                  intermediate_size=d.intermediate_size, n_quantizers=d.n_quantizers, codebook_size=d.codebook_size,
                  use_rq_transformer=True, rq_d_model=d.rq_d_model, rq_n_layers=d.rq_n_layers,
                  rq_n_heads=d.rq_n_heads, rope_dim=d.rope_dim, rope_theta=d.rope_theta,
                  rope_theta_rescale_factor=d.rope_theta_rescale_factor, vocab_size=d.vocab_size,
                  window_size=d.window_size, global_every=d.global_every, global_rope_dim=d.global_rope_dim,
                  global_rope_theta=d.global_rope_theta)
    cfg = Config(model=m, data=DataConfig(max_secs=0))
    # decoder.max_seqlen = max_text_tokens + max_audio_tokens + Q when data.max_secs gives 0 (model.py:1069-1073,1127)
    S = max_seqlen or d.max_seqlen
    m.max_text_tokens = S - d.n_quantizers
    m.max_audio_tokens = 0
    return cfg


def tiny_dims(kv=2, **kw):
    base = dict(d_model=64, n_layers=2, n_heads=4, n_kv_heads=kv, n_quantizers=4, codebook_size=32,
                rq_d_model=48, rq_n_layers=2, rq_n_heads=4, vocab_size=50, max_seqlen=32)
    base.update(kw)
    return O.Dims(**base)


TINY_SD = dict(seed=7, std=0.15, norm_jitter=0.1, bias_std=0.1)


def make_model(d: O.Dims, sd, dtype, int8=False, max_seqlen=None):
    from vui_amd.model import Vui

    return Vui(dims_to_config(d, max_seqlen), sd, device="cuda", dtype=dtype, int8=int8)


def rel_err(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.float().cpu(), b.float().cpu()
    return float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))
