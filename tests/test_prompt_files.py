"""Prompt files and checkpoint files (reference: tts_worker.py:885-1056, model.py:1154-1219)."""
import json
import types

import pytest
import torch

from oracle import vui_oracle as O
from tests.util import TINY_SD, dims_to_config, tiny_dims
from vui_amd import prompt as P


def test_match_n_q():
    c = torch.arange(12).view(3, 4)
    assert torch.equal(P.match_n_q(c, 4), c)
    assert torch.equal(P.match_n_q(c, 2), c[:, :2])
    p = P.match_n_q(c, 6)
    assert p.shape == (3, 6) and torch.equal(p[:, :4], c) and int(p[:, 4:].abs().sum()) == 0


class _FakeCache:
    def __init__(self, slots, S, KV, hd):
        self.k_cache = torch.zeros(slots, S, KV, hd)
        self.v_cache = torch.zeros(slots, S, KV, hd)


class _FakeRow:
    def __init__(self, eng):
        self.idx, self._eng, self._prompt_offset = 0, eng, 0

    @property
    def offset(self):
        return int(self._eng.seq_lens[0])

    def reset(self):
        self._eng.seq_lens[0] = 0


def _fake_engine(d_model=8, L=2, KV=2, hd=4, S=16, Q=4):
    caches = [_FakeCache(2, S, KV, hd) for _ in range(L)]
    model = types.SimpleNamespace(decoder=types.SimpleNamespace(flash_kv_caches=caches),
                                  config=types.SimpleNamespace(model=types.SimpleNamespace(d_model=d_model)),
                                  _cond_bias=torch.zeros(1, 1, d_model))
    eng = types.SimpleNamespace(model=model, Q=Q, seq_lens=torch.zeros(2, dtype=torch.int32), device="cpu")
    return eng, _FakeRow(eng)


def test_pt_prompt_round_trip_and_layout(tmp_path):
    eng, row = _fake_engine()
    g = torch.Generator().manual_seed(0)
    for c in eng.model.decoder.flash_kv_caches:
        c.k_cache.copy_(torch.randn(c.k_cache.shape, generator=g))
        c.v_cache.copy_(torch.randn(c.v_cache.shape, generator=g))
    eng.seq_lens[0] = 5
    eng.model._cond_bias.fill_(0.25)
    codes = torch.randint(0, 9, (7, 4), generator=g)
    f = str(tmp_path / "voice.pt")
    P.save_kv(f, eng, row, name="v", codes=codes, text="hello", checkpoint="ck1", spk_token_emb=torch.ones(1, 1, 8))
    # the layout the reference's loader reads (tts_worker.py:941-1000)
    raw = torch.load(f, weights_only=True)
    assert set(raw) == {"name", "codes", "text", "T", "n_q", "d_model", "checkpoint", "kv", "cond_bias", "spk_token_emb"}
    assert raw["T"] == 5 and raw["n_q"] == 4 and raw["d_model"] == 8 and len(raw["kv"]) == 2
    assert raw["kv"][0]["k"].shape == (1, 5, 2, 4) and raw["cond_bias"].shape == (1, 1, 8)
    want_k = [c.k_cache[0, :5].clone() for c in eng.model.decoder.flash_kv_caches]
    # restore into a clean engine
    eng2, row2 = _fake_engine()
    got = P.load_kv(f, eng2, row2, checkpoint="ck1")
    assert not got.needs_reprefill and got.T == 5 and got.name == "v" and got.text == "hello"
    assert row2.offset == 5 and row2._prompt_offset == 5
    for c, k in zip(eng2.model.decoder.flash_kv_caches, want_k):
        assert torch.equal(c.k_cache[0, :5], k) and float(c.k_cache[0, 5:].abs().sum()) == 0
        assert float(c.k_cache[1].abs().sum()) == 0  # the padding slot is untouched
    assert torch.equal(eng2.model._cond_bias, torch.full((1, 1, 8), 0.25))
    assert torch.equal(got.codes, codes) and torch.equal(got.spk_token_emb, torch.ones(1, 1, 8))
    # older files stored (1, KV, T, hd)
    raw["kv"] = [{"k": e["k"].transpose(1, 2).contiguous(), "v": e["v"].transpose(1, 2).contiguous()} for e in raw["kv"]]
    f2 = str(tmp_path / "old.pt")
    torch.save(raw, f2)
    eng3, row3 = _fake_engine()
    P.load_kv(f2, eng3, row3)
    assert torch.equal(eng3.model.decoder.flash_kv_caches[1].k_cache[0, :5], want_k[1])


def test_pt_prompt_stale_and_mismatch(tmp_path):
    eng, row = _fake_engine()
    eng.seq_lens[0] = 3
    f = str(tmp_path / "p.pt")
    P.save_kv(f, eng, row, name="p", codes=torch.zeros(2, 4, dtype=torch.long), checkpoint="a")
    e2, r2 = _fake_engine()
    got = P.load_kv(f, e2, r2, checkpoint="b")
    assert got.needs_reprefill and "checkpoint" in got.reason and r2.offset == 0
    got = P.load_kv(f, e2, r2, n_q=2)
    assert got.needs_reprefill and got.codes.shape == (2, 2)
    e3, r3 = _fake_engine(d_model=16)
    with pytest.raises(ValueError, match="d_model"):
        P.load_kv(f, e3, r3)
    e4, r4 = _fake_engine(hd=8)
    with pytest.raises(ValueError, match="head_dim"):
        P.load_kv(f, e4, r4)


def test_portable_prompt(tmp_path):
    eng, _ = _fake_engine()
    f = str(tmp_path / "p.safetensors")
    codes = torch.arange(12).view(2, 6)
    P.save_prompt_safetensors(f, name="n", codes=codes, text="t", cond_bias=torch.ones(1, 1, 8), d_model=8)
    got = P.load_kv(f, eng, None)
    assert got.needs_reprefill and got.name == "n" and got.text == "t" and torch.equal(got.codes, codes[:, :4])
    from safetensors import safe_open
    with safe_open(f, framework="pt") as h:  # the reference's reader: metadata "config" JSON + tensors by name
        assert json.loads(h.metadata()["config"]) == {"d_model": 8, "text": "t", "name": "n"}
        assert set(h.keys()) == {"codes", "cond_bias"}
    e2, _ = _fake_engine(d_model=4)
    with pytest.raises(ValueError, match="d_model"):
        P.load_kv(f, e2, None)


@pytest.mark.gpu
def test_checkpoint_files_and_prompt_restore(tmp_path):
    """A safetensors checkpoint with the config in its metadata and a torch checkpoint load into the
    same model (optional projections found from the keys); a saved prompt restored into a fresh
    engine continues exactly like the engine that prefilled it."""
    import dataclasses

    from safetensors.torch import save_file
    from tests.util import make_model
    from vui_amd.engine import Engine, GenConfig
    from vui_amd.model import Vui

    d = tiny_dims(max_seqlen=128)
    sd = O.synthetic_state_dict(d, **TINY_SD)
    cfg = dims_to_config(d, 128)
    cfgd = {"checkpoint": None, "model": dataclasses.asdict(cfg.model), "data": dataclasses.asdict(cfg.data)}
    cfgd["model"].pop("has_spk_proj", None)  # an older config without the flag
    sd2 = {**sd, "spk_proj.weight": torch.zeros(d.d_model, 16)}
    f_st = str(tmp_path / "m.safetensors")
    save_file({k: v.contiguous() for k, v in sd2.items()}, f_st, metadata={"config": json.dumps(cfgd)})
    f_pt = str(tmp_path / "m.pt")
    torch.save({"config": cfgd, "model": {"module." + k: v for k, v in sd2.items()}}, f_pt)
    m1 = Vui.from_pretrained(f_st, dtype=torch.float32)
    m2 = Vui.from_pretrained(f_pt, dtype=torch.float32)
    assert m1.config.model.has_spk_proj and m2.config.model.has_spk_proj
    with pytest.raises(FileNotFoundError):
        Vui.from_pretrained(str(tmp_path / "missing.safetensors"))

    g = torch.Generator().manual_seed(5)
    emb = (torch.randn(1, 9, d.d_model, generator=g) * 0.5).cuda()
    outs = []
    for m in (m1, m2):
        eng = Engine(model=m, max_rows=1, max_seq=128)
        row = eng.new_row()
        h = row.prefill_emb(emb)[:, -1]
        outs.append((eng, row, h))
    assert torch.equal(outs[0][2], outs[1][2])
    eng, row, h = outs[0]
    f = str(tmp_path / "voice.pt")
    P.save_kv(f, eng, row, name="voice", codes=torch.zeros(3, d.n_quantizers, dtype=torch.long), text="x")
    gc = GenConfig(top_k=1, rep_penalty=1.0)
    want, _ = eng.generate([row], h, 6, gc)
    eng3 = Engine(model=make_model(d, sd, torch.float32, max_seqlen=128), max_rows=1, max_seq=128)
    row3 = eng3.new_row()
    got = P.load_kv(f, eng3, row3)
    assert got.T == 9 and row3.offset == 9 and not got.needs_reprefill
    have, _ = eng3.generate([row3], h, 6, gc)
    assert torch.equal(want, have)
    # rewind returns to the end of the restored prompt
    assert row3.rewind() == 9
