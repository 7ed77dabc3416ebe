"""Model configuration.  Field names and defaults mirror the reference's pydantic schema
(src/vui/config.py:16-76) so a checkpoint's `config` dict can be passed through unchanged;
plain dataclasses are used, unknown keys are ignored like the reference's extra="ignore"."""
from __future__ import annotations

from dataclasses import dataclass, field, fields


def _from_dict(cls, d: dict):
    names = {f.name for f in fields(cls)}
    return cls(**{k: v for k, v in (d or {}).items() if k in names})


@dataclass
class VuiConfig:
    # Architecture
    d_model: int = 512
    n_layers: int = 6
    n_heads: int = 8
    n_kv_heads: int | None = None
    intermediate_size: int | None = None
    bias: bool = False
    dropout: float = 0.0
    max_text_tokens: int = 100
    max_audio_tokens: int = 100
    sinusoidal_cond: bool = False
    spk_emb_dim: int = 1024
    codec_hz: float = 12.5
    # RoPE
    use_rotary_emb: bool = True
    rope_dim: int | None = None
    rope_theta: float = 10_000.0
    rope_theta_rescale_factor: float = 1.0
    global_rope_dim: int | None = None
    global_rope_theta: float | None = None
    window_size: int | None = None
    global_every: int | None = None
    # RQ-Transformer head
    use_rq_transformer: bool = False
    rq_d_model: int = 512
    rq_n_layers: int = 6
    rq_n_heads: int = 6
    n_quantizers: int = 9
    codebook_size: int = 4096
    # Conditioning projection heads
    has_sq_proj: bool = False
    has_wps_proj: bool = False
    has_spk_proj: bool = False
    # The reference takes the text vocabulary size from its tokenizer (src/vui/model.py:1075-1076);
    # without a tokenizer it is carried here (and otherwise read off token_emb.weight).
    vocab_size: int = 0

    @property
    def head_dim(self) -> int:
        return self.d_model // self.n_heads

    @property
    def kv_heads(self) -> int:
        return self.n_kv_heads if self.n_kv_heads is not None else self.n_heads

    @property
    def ffn(self) -> int:
        """LlamaMLP hidden size, src/vui/model.py:272-277."""
        if self.intermediate_size is not None:
            return self.intermediate_size
        h = int(2 * (4 * self.d_model) / 3)
        return 256 * ((h + 255) // 256)

    @property
    def rq_ffn(self) -> int:
        """RQBlock hidden size, src/vui/model.py:587-588."""
        h = int(self.rq_d_model * 8 / 3)
        return 64 * ((h + 63) // 64)


@dataclass
class DataConfig:
    max_secs: float = 360


@dataclass
class Config:
    checkpoint: str | dict | None = None
    model: VuiConfig = field(default_factory=VuiConfig)
    data: DataConfig = field(default_factory=DataConfig)

    @property
    def max_seq_len(self) -> int:
        """src/vui/config.py:70-76."""
        audio_tokens = int(self.data.max_secs * self.model.codec_hz)
        text_tokens = int(audio_tokens * 2.5)
        total = audio_tokens + text_tokens
        return 64 * ((total + 63) // 64)

    @classmethod
    def from_dict(cls, d: dict) -> "Config":
        return cls(checkpoint=d.get("checkpoint"), model=_from_dict(VuiConfig, d.get("model")),
                   data=_from_dict(DataConfig, d.get("data")))


def nano_config(preset: str = "A", max_secs: float = 240) -> Config:
    """Vui Nano.  Backbone dims are documented by the reference (README.md:270-271,
    docs/memory-budget.md:43,131); the depth head's are not and only two round-number fits
    reach the documented 305 M parameters: A = 512-d x 4 layers with a 100554-token vocabulary,
    B = 768-d x 5 layers with a 50534-token one."""
    base = dict(d_model=768, n_layers=22, n_heads=8, n_kv_heads=8, n_quantizers=16, codebook_size=2048,
                use_rq_transformer=True, has_spk_proj=True)
    if preset.upper() == "A":
        m = VuiConfig(**base, rq_d_model=512, rq_n_layers=4, rq_n_heads=8, vocab_size=100554)
    elif preset.upper() == "B":
        m = VuiConfig(**base, rq_d_model=768, rq_n_layers=5, rq_n_heads=8, vocab_size=50534)
    else:
        raise ValueError(f"unknown preset {preset!r}")
    return Config(model=m, data=DataConfig(max_secs=max_secs))
