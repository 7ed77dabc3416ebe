"""Voice-prompt files: the prefilled KV cache of a row on disk, and the portable prompt.

Two formats of the reference's streaming worker (src/vui/serving/stream/tts_worker.py:885-1056):

* `.pt` -- `torch.save` of {"name", "codes" (T_audio, Q), "text", "T", "n_q", "d_model",
  "checkpoint", "kv": [{"k", "v"} per layer, each (1, T, KV, hd)], "cond_bias" (1, 1, d),
  "spk_token_emb" or None}.  Loading copies K/V straight into the row's cache slot and sets
  seq_lens: no recompute.  Files are read with `weights_only=True` (tensors and plain containers
  only; the reference unpickles).
* `.safetensors` -- tensors "codes", "cond_bias", optional "spk_token_emb"; metadata "config" =
  JSON {"d_model", "text", "name"}.  It carries no K/V: the prompt is prefilled again from codes
  and text, which needs the text embedder the caller owns.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass

import torch
from torch import Tensor


@dataclass
class LoadedPrompt:
    name: str
    codes: Tensor | None  # (T_audio, Q') matched to the model's n_q
    text: str
    T: int  # cache positions restored (0 when the prompt has to be prefilled again)
    spk_token_emb: Tensor | None
    cond_bias: Tensor | None
    needs_reprefill: bool
    reason: str = ""


def match_n_q(codes: Tensor, n_q: int) -> Tensor:
    """Trim or zero-pad the last dim of saved codes to n_q (tts_worker.py:915-928)."""
    q = codes.shape[-1]
    if q == n_q:
        return codes
    if q > n_q:
        return codes[..., :n_q].contiguous()
    return torch.nn.functional.pad(codes, (0, n_q - q)).contiguous()


def save_kv(path: str, engine, row, *, name: str, codes: Tensor | None = None, text: str = "", n_q: int | None = None,
            checkpoint: str | None = None, spk_token_emb: Tensor | None = None) -> None:
    """Writes the row's first `row.offset` cache positions in the reference's `.pt` layout
    (save_kv, tts_worker.py:885-913)."""
    T = row.offset
    i = row.idx
    kv = [{"k": c.k_cache[i:i + 1, :T].cpu().clone(), "v": c.v_cache[i:i + 1, :T].cpu().clone()}
          for c in engine.model.decoder.flash_kv_caches]
    torch.save({
        "name": name, "codes": codes, "text": text, "T": T, "n_q": n_q if n_q is not None else engine.Q,
        "d_model": engine.model.config.model.d_model, "checkpoint": checkpoint, "kv": kv,
        "cond_bias": engine.model._cond_bias.cpu().clone(),
        "spk_token_emb": spk_token_emb.cpu().clone() if spk_token_emb is not None else None,
    }, path)


def load_kv(path: str, engine, row, *, n_q: int | None = None, checkpoint: str | None = None) -> LoadedPrompt:
    """Restores a `.pt` prompt into the row (load_kv, tts_worker.py:941-1024) or reads a portable
    `.safetensors` one (:1026-1056).  Errors as the reference: ValueError on a d_model or head_dim
    mismatch.  A prompt saved with another checkpoint or another n_q is stale: nothing is copied
    and needs_reprefill is set (the caller prefills from codes and text)."""
    if str(path).endswith(".safetensors"):
        return load_prompt_safetensors(path, engine)
    saved = torch.load(path, map_location="cpu", weights_only=True)
    n_q = n_q if n_q is not None else engine.Q
    mcfg = engine.model.config.model
    saved_d = saved.get("d_model", 0)
    if saved_d and saved_d != mcfg.d_model:
        raise ValueError(f"KV cache d_model mismatch: saved={saved_d}, model={mcfg.d_model}")
    codes = saved.get("codes")
    saved_nq = saved.get("n_q") or (int(codes.shape[-1]) if codes is not None else 0)
    saved_ckpt = saved.get("checkpoint")
    reasons = []
    if saved_nq and saved_nq != n_q:
        reasons.append(f"n_q {saved_nq}->{n_q}")
    if saved_ckpt and checkpoint and saved_ckpt != checkpoint:
        reasons.append("checkpoint changed")
    name = saved.get("name", os.path.splitext(os.path.basename(str(path)))[0])
    spk = saved.get("spk_token_emb")
    matched = match_n_q(codes, n_q) if codes is not None else None
    if reasons:
        return LoadedPrompt(name, matched, saved.get("text", ""), 0, spk, saved["cond_bias"], True, ", ".join(reasons))
    caches = engine.model.decoder.flash_kv_caches
    if saved["kv"][0]["k"].shape[-1] != caches[0].k_cache.shape[-1]:
        raise ValueError(f"KV cache head_dim mismatch: saved={saved['kv'][0]['k'].shape[-1]}, "
                         f"model={caches[0].k_cache.shape[-1]}")
    if len(saved["kv"]) != len(caches):
        raise ValueError(f"KV cache layer count mismatch: saved={len(saved['kv'])}, model={len(caches)}")
    T = int(saved["T"])
    if T > caches[0].k_cache.shape[1]:
        raise ValueError(f"prompt of {T} positions exceeds the cache length {caches[0].k_cache.shape[1]}")
    row.reset()
    engine.model._cond_bias.copy_(saved["cond_bias"].to(engine.model._cond_bias.device))
    i = row.idx
    for c, kv_saved in zip(caches, saved["kv"]):
        k, v = kv_saved["k"], kv_saved["v"]
        n_kv = c.k_cache.shape[2]
        if k.dim() == 4 and k.shape[1] == n_kv and k.shape[2] == T and n_kv != T:  # older (1, KV, T, hd) files
            k, v = k.transpose(1, 2), v.transpose(1, 2)
        c.k_cache[i:i + 1, :T].copy_(k[:1].to(c.k_cache.device, c.k_cache.dtype))
        c.v_cache[i:i + 1, :T].copy_(v[:1].to(c.v_cache.device, c.v_cache.dtype))
    engine.seq_lens[i] = T
    row._prompt_offset = T
    return LoadedPrompt(name, matched, saved.get("text", ""), T, spk.to(engine.device) if spk is not None else None,
                        saved["cond_bias"], False)


def save_prompt_safetensors(path: str, *, name: str, codes: Tensor, text: str, cond_bias: Tensor, d_model: int,
                            spk_token_emb: Tensor | None = None) -> None:
    from safetensors.torch import save_file

    tensors = {"codes": codes.contiguous().cpu(), "cond_bias": cond_bias.contiguous().cpu()}
    if spk_token_emb is not None:
        tensors["spk_token_emb"] = spk_token_emb.contiguous().cpu()
    save_file(tensors, path, metadata={"config": json.dumps({"d_model": d_model, "text": text, "name": name})})


def load_prompt_safetensors(path: str, engine) -> LoadedPrompt:
    """tts_worker.py:1026-1056: always a re-prefill from codes and text."""
    from safetensors import safe_open

    with safe_open(path, framework="pt") as f:
        cfg = json.loads((f.metadata() or {}).get("config", "{}"))
        tensors = {k: f.get_tensor(k) for k in f.keys()}
    d_model = engine.model.config.model.d_model
    saved_d = int(cfg.get("d_model", 0))
    if saved_d and saved_d != d_model:
        raise ValueError(f"Prompt d_model mismatch: saved={saved_d}, model={d_model}")
    name = cfg.get("name", os.path.splitext(os.path.basename(str(path)))[0])
    return LoadedPrompt(name, match_n_q(tensors["codes"], engine.Q), cfg.get("text", ""), 0, tensors.get("spk_token_emb"),
                        tensors["cond_bias"], True, "portable prompt")
