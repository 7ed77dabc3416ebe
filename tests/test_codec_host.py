"""Host-side vocoder logic without a GPU: CodecCtx bookkeeping of the package against the oracle's
restatement (both driven by the same recording stand-in decoder), the checkpoint key map, the
state-dict layout and the C-ABI size queries."""
import ctypes as C
import dataclasses

import pytest
import torch

from oracle import codec_oracle as O
from vui_amd import codec as K


class FakeStream:
    def __init__(self, dec):
        self.dec = dec

    def close(self):
        self.dec.log.append(("close",))
        self.dec._streaming = False


class FakeDecoder:
    """Records what a CodecCtx asks of its decoder; audio = frame count so far."""

    hop = 4

    def __init__(self):
        self.log = []
        self._streaming = False

    # package surface
    def streaming(self, n=1):
        self.log.append(("open",))
        self._streaming = True
        return FakeStream(self)

    def __call__(self, codes):
        self.log.append(("decode", tuple(codes.shape), int(codes.sum())))
        return torch.zeros(1, 1, codes.shape[2] * self.hop)

    # oracle surface
    def open_stream(self):
        self.log.append(("open",))

    def close_stream(self):
        self.log.append(("close",))

    forward = __call__


def drive(ctx, frames=300):
    g = torch.Generator().manual_seed(0)
    ctx.set_prompt(torch.randint(0, 9, (1, 16, 37), generator=g))
    ctx.add(torch.randint(0, 9, (16, 20), generator=g))
    ctx.prefill(n_codebooks=8)
    fsp = []
    for t in range(frames):
        c = torch.randint(0, 9, (1, 16, 1), generator=g)
        ctx.decode_frame(c[:, :8], store_codes=c)
        fsp.append((ctx._frames_since_prefill, ctx.n_frames))
    ctx.reset()
    return fsp


def test_codec_ctx_equals_oracle_restatement():
    a, b = FakeDecoder(), FakeDecoder()
    fa = drive(K.CodecCtx(a))
    fb = drive(O.CodecCtxOracle(b))
    assert fa == fb
    assert a.log == b.log
    # seeding: 57 buffered frames -> the last 57 % 125 with 8 codebooks; restart after 125 frames
    assert a.log[0] == ("open",) and a.log[1][1] == (1, 8, 57)
    opens = [i for i, e in enumerate(a.log) if e == ("open",)]
    assert len(opens) == 1 + 2  # prefill, then two cold restarts within 300 frames (at 68 and 193)
    assert fa[67][0] == 125 and fa[68][0] == 1
    assert max(n for _, n in fa) == 250  # the buffer is capped at two windows, the prompt kept


def test_codec_ctx_full_decode_windows():
    d = FakeDecoder()
    ctx = K.CodecCtx(d)
    ctx.set_prompt(torch.zeros(1, 16, 30, dtype=torch.long))
    out = ctx(torch.ones(1, 16, 10, dtype=torch.long))
    assert out.shape[-1] == 10 * d.hop and d.log[-1][1] == (1, 16, 40)
    out = ctx(torch.ones(1, 16, 200, dtype=torch.long))  # longer than a window: chunks with half-window context
    assert out.shape[-1] == 200 * d.hop
    assert all(e[1][2] <= ctx.max_ctx for e in d.log if e[0] == "decode")
    assert ctx.n_frames == 240


def test_state_dict_layout_matches_oracle():
    for d in (O.CodecDims(), O.tiny_dims()):
        cfg = K.CodecConfig(**dataclasses.asdict(d))
        assert list(K.codec_state_dict_shapes(cfg).items()) == list(O.codec_state_dict_shapes(d).items())
        assert cfg.hop == d.hop
    assert K.CodecConfig().hop == 1920


def test_hf_key_map():
    """Key names of the published checkpoint (qwen_codec.py:1391-1480): spot checks of every renamed family."""
    m = K.hf_key_map(K.CodecConfig())
    assert m["pre_transformer.layers.3.q_proj.weight"] == "pre_transformer.layers.3.self_attn.q_proj.weight"
    assert m["pre_transformer.layers.0.attn_scale"] == "pre_transformer.layers.0.self_attn_layer_scale.scale"
    assert m["pre_transformer.layers.7.mlp_scale"] == "pre_transformer.layers.7.mlp_layer_scale.scale"
    assert m["pre_transformer.layers.7.down_proj.weight"] == "pre_transformer.layers.7.mlp.down_proj.weight"
    assert m["pre_transformer.layers.1.input_layernorm.weight"] == "pre_transformer.layers.1.input_layernorm.weight"
    assert m["quantizer.semantic.output_proj.weight"] == "quantizer.rvq_first.output_proj.weight"
    assert m["quantizer.acoustic.output_proj.weight"] == "quantizer.rvq_rest.output_proj.weight"
    assert m["decoder.3.block.2.conv1.conv.weight"] == "decoder.3.block.2.conv1.conv.weight"
    assert m["upsample.1.1.gamma"] == "upsample.1.1.gamma"
    assert not any("codebooks" in k for k in m)
    assert len(m) == 255 - 16 - 2


def test_abi_size_queries():
    from vui_amd import _lib

    lib = _lib.load()
    c = K.CodecConfig().to_c()
    assert lib.vui_codec_hop(C.byref(c)) == 1920
    assert lib.vui_codec_n_tensors(C.byref(c)) == 255 == len(K.codec_state_dict_shapes(K.CodecConfig()))
    need = lib.vui_codec_workspace_bytes(C.byref(c))
    assert 460e6 < need < 520e6  # 457 MB of repacked fp32 weights + 33.5 MB of codebooks... minus what is folded
    bad = K.CodecConfig(latent_dim=24).to_c()
    assert lib.vui_codec_workspace_bytes(C.byref(bad)) < 0 and "multiple of 32" in _lib.last_error()
    bad = K.CodecConfig(head_dim=40, n_heads=8).to_c()
    assert lib.vui_codec_hop(C.byref(bad)) < 0 and "head_dim" in _lib.last_error()
    h = C.c_void_p()
    assert lib.vui_codec_init(C.byref(c), None, 255, None, 0, None, C.byref(h)) == -22
    assert lib.vui_codec_decode_frame(None, None, 16, None, None) == -22 and "NULL codec" in _lib.last_error()
