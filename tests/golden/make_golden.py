"""Writes the golden vectors under tests/golden/ from the reference's own classes.

Run once, in the build container only (the reference checkout does not travel):

    PYTHONPATH=/root/reference/src python tests/golden/make_golden.py [--skip-nano]

It imports the reference's `vui.model`, `vui.rope` and `vui.sampling`, loads deterministic
synthetic weights (oracle.vui_oracle.synthetic_state_dict) into the reference modules and
records small input/output vectors as .npz files.  The fixtures are data only.

Fixtures:
  rope.npz        precompute_freqs_cis (plain and rescaled/partial) + apply_rotary_emb
  pieces.npz      RMSNorm, AudioEmbedding (incl. Q' < Q), sample_top_k support/histogram
  tiny_backbone_{mha,gqa}.npz   Decoder.forward (SDPA + KVCache): prefill T=5, then 4 decode steps
  tiny_backbone_global_{a,b,c}.npz   Decoder.forward with window_size / global_every / global_rope_* set: which
                  layers are global, their own rotation table, prefill T=9 and 4 decode steps
  tiny_rq.npz     RQTransformer.forward logits, generate(top_k=1) codes, top-k sampling histogram
  tiny_bf16.npz   the same tiny decoder and RQ head run in bfloat16 on CPU
  nano_grid.npz   the full-size greedy 64x16 token grid with fp32 weights N(0,0.02), seed 0
"""
import argparse
import os
import sys
import time

import numpy as np
import torch
import torch.nn as nn

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle.vui_oracle import Dims, synthetic_state_dict  # noqa: E402

import vui.model as M  # noqa: E402  (reference)
import vui.rope as R  # noqa: E402  (reference)
import vui.sampling as S  # noqa: E402  (reference)


def sub(sd, prefix):
    return {k[len(prefix):]: v for k, v in sd.items() if k.startswith(prefix)}


def build_reference(d: Dims, sd, max_seqlen: int, dtype=torch.float32):
    """Reference modules wired as Vui.__init__ does (model.py:1076-1136), minus the tokenizer."""
    dec = M.Decoder(n_layers=d.n_layers, d_model=d.d_model, n_heads=d.n_heads, n_kv_heads=d.n_kv_heads,
                    bias=False, dropout=0.0, max_seqlen=max_seqlen, rope_dim=d.rope_dim,
                    rope_theta=d.rope_theta, rope_theta_rescale_factor=d.rope_theta_rescale_factor,
                    intermediate_size=d.intermediate_size, window_size=d.window_size, global_every=d.global_every,
                    global_rope_dim=d.global_rope_dim, global_rope_theta=d.global_rope_theta)
    dec.load_state_dict(sub(sd, "decoder."), strict=True)
    aemb = M.AudioEmbedding(d.n_quantizers, d.codebook_size, d.d_model)
    aemb.load_state_dict(sub(sd, "audio_emb."), strict=True)
    temb = nn.Embedding(d.vocab_size, d.d_model)
    temb.load_state_dict(sub(sd, "token_emb."), strict=True)
    chead = nn.Linear(d.d_model, d.codebook_size, bias=False)
    chead.load_state_dict(sub(sd, "codec_head."), strict=True)
    ehead = nn.Linear(d.d_model, 1)
    ehead.load_state_dict(sub(sd, "eos_head."), strict=True)
    rq = M.RQTransformer(backbone_dim=d.d_model, rq_dim=d.rq_d_model, n_layers=d.rq_n_layers,
                         n_heads=d.rq_n_heads, n_quantizers=d.n_quantizers, codebook_size=d.codebook_size)
    rq.load_state_dict(sub(sd, "rq_transformer."), strict=True)
    mods = dict(dec=dec, aemb=aemb, temb=temb, chead=chead, ehead=ehead, rq=rq)
    for m in mods.values():
        m.to(dtype).eval()
    # SDPA path: per-block KVCache + a causal mask indexed by input_pos (model.py:42-68,182-198,514-518)
    for blk in dec.blocks:
        blk.attn.kv_cache = M.KVCache(1, max_seqlen, d.n_kv_heads, d.head_dim, dtype=dtype)
    dec.attn_mask = torch.tril(torch.ones(max_seqlen, max_seqlen, dtype=torch.bool))
    return mods


def tiny_dims(kv):
    return Dims(d_model=64, n_layers=2, n_heads=4, n_kv_heads=kv, n_quantizers=4, codebook_size=32,
                rq_d_model=48, rq_n_layers=2, rq_n_heads=4, vocab_size=50, max_seqlen=32)


TINY_SD = dict(seed=7, std=0.15, norm_jitter=0.1, bias_std=0.1)


@torch.inference_mode()
def make_rope():
    out = {}
    out["plain"] = R.precompute_freqs_cis(96, 40).numpy()
    out["rescaled"] = R.precompute_freqs_cis(8, 24, theta=500.0, theta_rescale_factor=1.7).numpy()
    g = torch.Generator().manual_seed(1)
    t = torch.randn(2, 3, 5, 16, generator=g)  # (B, heads, T, hd)
    fr_full = R.precompute_freqs_cis(16, 24)[torch.tensor([3, 4, 9, 10, 23])]
    fr_part = R.precompute_freqs_cis(8, 24, theta=500.0, theta_rescale_factor=1.7)[torch.tensor([3, 4, 9, 10, 23])]
    out["t"] = t.numpy()
    out["pos"] = np.array([3, 4, 9, 10, 23])
    out["rot_full"] = R.apply_rotary_emb(fr_full, t).numpy()
    out["rot_part"] = R.apply_rotary_emb(fr_part, t).numpy()
    # per-sample (3-dim) form used at decode: t (B, heads, hd), freqs (B, rot, 2)  (model.py:235-237)
    t3 = torch.randn(5, 3, 16, generator=g)
    out["t3"] = t3.numpy()
    out["rot3"] = R.apply_rotary_emb(fr_full, t3).numpy()
    out["rot3_bf16"] = R.apply_rotary_emb(fr_full, t3.bfloat16()).float().numpy()
    np.savez_compressed(os.path.join(HERE, "rope.npz"), **out)


@torch.inference_mode()
def make_pieces():
    out = {}
    g = torch.Generator().manual_seed(2)
    x = torch.randn(3, 2, 24, generator=g) * 3
    n = M.RMSNorm(24, eps=1e-5)
    n.weight.copy_(1 + 0.3 * torch.randn(24, generator=g))
    out["norm_x"] = x.numpy()
    out["norm_w"] = n.weight.detach().numpy()
    out["norm_y"] = n(x).numpy()
    nb = M.RMSNorm(24, eps=1e-5).bfloat16()
    nb.weight.copy_(n.weight.bfloat16())
    out["norm_y_bf16"] = nb(x.bfloat16()).float().numpy()
    ae = M.AudioEmbedding(4, 8, 6)
    ae.embedding.weight.copy_(torch.randn(32, 6, generator=g))
    codes = torch.randint(0, 8, (5, 4), generator=g)
    out["ae_table"] = ae.embedding.weight.detach().numpy()
    out["ae_codes"] = codes.numpy()
    out["ae_full"] = ae(codes).numpy()
    out["ae_q2"] = ae(codes[:, :2]).numpy()
    # sample_top_k (sampling.py:14-20): support and histogram over many draws, with a tie at the k-th place
    p = torch.tensor([0.02, 0.2, 0.1, 0.1, 0.3, 0.1, 0.05, 0.13])
    torch.manual_seed(3)
    draws = S.sample_top_k(p.repeat(40000, 1), 3).squeeze(-1)
    out["tk_probs"] = p.numpy()
    out["tk_k"] = np.array(3)
    out["tk_hist"] = torch.bincount(draws, minlength=8).numpy()
    np.savez_compressed(os.path.join(HERE, "pieces.npz"), **out)


@torch.inference_mode()
def run_backbone(mods, d, ids, codes_seq):
    """prefill the text ids, then feed the given code frames one by one (T=1)."""
    dec = mods["dec"]
    T = ids.shape[0]
    x = mods["temb"](ids[None])
    h_pre = dec(x, torch.arange(T))
    outs_h, outs_cb0, outs_eos = [], [], []
    pos = T
    for fr in codes_seq:
        emb = mods["aemb"](fr[None])[None]  # (1,1,d)
        h = dec(emb, torch.tensor([pos]))[:, 0]
        pos += 1
        outs_h.append(h[0])
        outs_cb0.append(mods["chead"](h)[0])
        outs_eos.append(mods["ehead"](h)[0])
    return h_pre[0], torch.stack(outs_h), torch.stack(outs_cb0), torch.stack(outs_eos)


@torch.inference_mode()
def make_tiny_backbone(kv, name):
    d = tiny_dims(kv)
    sd = synthetic_state_dict(d, **TINY_SD)
    mods = build_reference(d, sd, d.max_seqlen)
    g = torch.Generator().manual_seed(11)
    ids = torch.randint(0, d.vocab_size, (5,), generator=g)
    codes_seq = torch.randint(0, d.codebook_size, (4, d.n_quantizers), generator=g)
    h_pre, h, cb0, eos = run_backbone(mods, d, ids, codes_seq)
    k0 = mods["dec"].blocks[0].attn.kv_cache.k_cache[0, :, :9].numpy()  # (KV, 9, hd)
    v1 = mods["dec"].blocks[1].attn.kv_cache.v_cache[0, :, :9].numpy()
    np.savez_compressed(os.path.join(HERE, name), ids=ids.numpy(), codes=codes_seq.numpy(),
                        h_prefill=h_pre.numpy(), hidden=h.numpy(), cb0=cb0.numpy(), eos=eos.numpy(),
                        k_layer0=k0, v_layer1=v1)


@torch.inference_mode()
def make_tiny_backbone_global():
    """Decoder with a window, global-attention layers and their own rotation table (model.py:396-468, 504-509):
    which layers are global, the derived table, and forward outputs.  The reference's CPU path (SDPA + KVCache)
    applies no window (only flash-attn does, model.py:256), so these vectors pin which table rotates which layer."""
    for name, kw in (("a", dict(n_layers=3, window_size=6, global_every=2, global_rope_dim=8)),
                     ("b", dict(n_layers=4, window_size=8, global_every=3)),
                     ("c", dict(n_layers=2, global_rope_theta=500.0))):
        d = tiny_dims(2)
        for k, v in kw.items():
            setattr(d, k, v)
        sd = synthetic_state_dict(d, **TINY_SD)
        mods = build_reference(d, sd, d.max_seqlen)
        dec = mods["dec"]
        g = torch.Generator().manual_seed(21)
        ids = torch.randint(0, d.vocab_size, (9,), generator=g)
        codes_seq = torch.randint(0, d.codebook_size, (4, d.n_quantizers), generator=g)
        h_pre, h, cb0, eos = run_backbone(mods, d, ids, codes_seq)
        out = dict(ids=ids.numpy(), codes=codes_seq.numpy(), h_prefill=h_pre.numpy(), hidden=h.numpy(), cb0=cb0.numpy(),
                   is_global=np.array(dec.block_is_global), kw_keys=np.array(sorted(kw)),
                   kw_vals=np.array([float(kw[k]) for k in sorted(kw)]))
        if dec.freqs_cis_global is not None:
            out["freqs_global"] = dec.freqs_cis_global.numpy()
        np.savez_compressed(os.path.join(HERE, f"tiny_backbone_global_{name}.npz"), **out)


@torch.inference_mode()
def make_tiny_rq():
    d = tiny_dims(4)
    sd = synthetic_state_dict(d, **TINY_SD)
    mods = build_reference(d, sd, d.max_seqlen)
    rq = mods["rq"]
    g = torch.Generator().manual_seed(12)
    hidden = torch.randn(3, d.d_model, generator=g)
    codes = torch.randint(0, d.codebook_size, (3, d.n_quantizers), generator=g)
    out = dict(hidden=hidden.numpy(), codes=codes.numpy())
    out["forward_logits"] = rq(hidden, codes).numpy()
    out["forward_logits_q3"] = rq(hidden, codes[:, :3]).numpy()
    out["greedy"] = rq.generate(hidden, codes[:, 0], temperature=1.0, top_k=1).numpy()
    bias = 0.5 * torch.randn(d.n_quantizers - 1, d.codebook_size, generator=g)
    out["bias"] = bias.numpy()
    out["greedy_bias"] = rq.generate(hidden, codes[:, 0], temperature=0.7, top_k=1, logit_bias=bias).numpy()
    # sampling: many identical rows -> histogram of the first sampled codebook, top_k=5, T=0.8
    torch.manual_seed(13)
    N = 20000
    samp = rq.generate(hidden[:1].repeat(N, 1), codes[:1, 0].repeat(N), temperature=0.8, top_k=5)
    out["samp_hist_cb1"] = torch.bincount(samp[:, 1], minlength=d.codebook_size).numpy()
    np.savez_compressed(os.path.join(HERE, "tiny_rq.npz"), **out)


@torch.inference_mode()
def make_tiny_bf16():
    d = tiny_dims(2)
    sd = synthetic_state_dict(d, **TINY_SD)
    mods = build_reference(d, sd, d.max_seqlen, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(11)
    ids = torch.randint(0, d.vocab_size, (5,), generator=g)
    codes_seq = torch.randint(0, d.codebook_size, (4, d.n_quantizers), generator=g)
    h_pre, h, cb0, eos = run_backbone(mods, d, ids, codes_seq)
    hidden = torch.randn(3, d.d_model, generator=g).bfloat16()
    rq_logits = mods["rq"](hidden, codes_seq[:3])
    np.savez_compressed(os.path.join(HERE, "tiny_bf16.npz"), ids=ids.numpy(), codes=codes_seq.numpy(),
                        h_prefill=h_pre.float().numpy(), hidden=h.float().numpy(), cb0=cb0.float().numpy(),
                        eos=eos.float().numpy(), rq_hidden=hidden.float().numpy(),
                        rq_logits=rq_logits.float().numpy())


def top2_margin(logits):
    v = torch.topk(logits.float(), 2, dim=-1).values
    return (v[..., 0] - v[..., 1])


@torch.inference_mode()
def make_nano_grid(n_frames=64, n_text=32):
    """Benchmark config 1: Vui Nano dims, fp32 weights N(0,0.02) seed 0, 32 uniform text ids,
    greedy decode of 64 frames x 16 codebooks.  Driver order follows inference.py:680-726:
    prefill -> code0 = argmax(codec_head(h_last)) -> rq.generate(top_k=1) -> decode step."""
    d = Dims()  # preset A
    t0 = time.time()
    sd = synthetic_state_dict(d, seed=0)
    S_len = 128
    mods = build_reference(d, sd, S_len)
    print(f"  built reference modules in {time.time()-t0:.1f}s", flush=True)
    g = torch.Generator().manual_seed(0)
    ids = torch.randint(0, d.vocab_size, (n_text,), generator=g)
    dec, rq = mods["dec"], mods["rq"]
    h = dec(mods["temb"](ids[None]), torch.arange(n_text))[:, -1]  # (1,d)
    first_hidden = h[0].clone()
    pos = n_text
    grid, margins_cb0, margins_rq, eos_all, cb0_first = [], [], [], [], None
    for f in range(n_frames):
        cb0 = mods["chead"](h)
        if f == 0:
            cb0_first = cb0[0].clone()
        eos_all.append(mods["ehead"](h)[0, 0])
        margins_cb0.append(top2_margin(cb0)[0])
        code0 = cb0.argmax(-1)
        frame = rq.generate(h, code0, temperature=1.0, top_k=1)  # (1,Q)
        # margins of the RQ logits along the greedy path (teacher-forced forward gives the same logits)
        margins_rq.append(top2_margin(rq(h, frame))[0])
        grid.append(frame[0])
        emb = mods["aemb"](frame)[None]  # (1,1,d)
        h = dec(emb, torch.tensor([pos]))[:, 0]
        pos += 1
        if f % 8 == 0:
            print(f"  frame {f} {frame[0].tolist()[:4]}... {time.time()-t0:.1f}s", flush=True)
    chk = {k: int(sd[k].view(torch.int32).to(torch.int64).sum()) for k in ("token_emb.weight", "decoder.blocks.21.mlp.w2.weight",
                                                   "rq_transformer.head_W")}
    np.savez_compressed(os.path.join(HERE, "nano_grid.npz"), ids=ids.numpy(), grid=torch.stack(grid).numpy(),
                        margin_cb0=torch.stack(margins_cb0).numpy(), margin_rq=torch.stack(margins_rq).numpy(),
                        eos=torch.stack(eos_all).numpy(), first_hidden=first_hidden.numpy(),
                        cb0_first=cb0_first.numpy(), last_hidden=h[0].numpy(),
                        weight_checksums=np.array([chk[k] for k in sorted(chk)]),
                        weight_checksum_keys=np.array(sorted(chk)))


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--skip-nano", action="store_true")
    ap.add_argument("--only-global", action="store_true", help="write only the global-attention-layer fixtures")
    a = ap.parse_args()
    torch.set_num_threads(8)
    if a.only_global:
        make_tiny_backbone_global()
        sys.exit(0)
    make_rope()
    make_pieces()
    make_tiny_backbone(4, "tiny_backbone_mha.npz")
    make_tiny_backbone(2, "tiny_backbone_gqa.npz")
    make_tiny_backbone_global()
    make_tiny_rq()
    make_tiny_bf16()
    print("small fixtures written", flush=True)
    if not a.skip_nano:
        make_nano_grid()
        print("nano grid written", flush=True)
