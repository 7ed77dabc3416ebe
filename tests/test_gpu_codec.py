"""The native vocoder frame step against the CPU oracle and against vectors written from the
reference's own classes (through the C ABI, fp32)."""
import dataclasses
import os

import numpy as np
import pytest
import torch

from oracle import codec_oracle as O

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")
TOL = 2e-4  # absolute, on audio in [-1, 1] (fp32 sums in another order through ~60 layers)


def small_dims():
    return O.CodecDims(n_codebooks=4, codebook_size=32, codebook_dim=16, vq_dim=32, latent_dim=64, d_model=32,
                       n_layers=2, n_heads=2, head_dim=16, mlp_dim=64, max_seq=40, up_ratios=(2, 2),
                       decoder_dim=128, rates=(3, 2))


def native(d, sd):
    from vui_amd.codec import CodecConfig, QwenCodecDecoder

    return QwenCodecDecoder(sd, CodecConfig(**dataclasses.asdict(d)), device="cuda")


@pytest.fixture(scope="module")
def small():
    d = small_dims()
    sd = O.synthetic_codec_state_dict(d, seed=4)
    return d, O.CodecDecoderOracle(d, sd), native(d, sd)


@pytest.fixture(scope="module")
def full():
    d = O.CodecDims()
    sd = O.synthetic_codec_state_dict(d, seed=0)
    fx = {k: torch.from_numpy(v) for k, v in np.load(os.path.join(GOLD, "codec_full.npz")).items()}
    return d, sd, native(d, sd), fx


def err(a, b):
    return float((a.detach().cpu().float() - b.float()).abs().max())


def test_small_stream_frame_by_frame(small):
    d, ora, dec = small
    g = torch.Generator().manual_seed(1)
    codes = torch.randint(0, d.codebook_size, (1, d.n_codebooks, 14), generator=g)
    ora.open_stream()
    with dec.streaming(1):
        for t in range(codes.shape[2]):
            ref = ora.forward(codes[:, :, t:t + 1])
            got = dec(codes[:, :, t:t + 1].cuda())
            assert got.shape == (1, 1, d.hop)
            assert err(got, ref) < TOL, (t, err(got, ref))
        assert dec.frames_since_reset() == 14
    ora.close_stream()
    assert float(ref.abs().max()) > 0.05  # the comparison is not about silence


def test_small_offline_chunk_and_fewer_codebooks(small):
    d, ora, dec = small
    g = torch.Generator().manual_seed(2)
    codes = torch.randint(0, d.codebook_size, (1, d.n_codebooks, 9), generator=g)
    assert err(dec(codes.cuda()), ora.forward(codes)) < TOL
    assert err(dec(codes[:, :2].cuda()), ora.forward(codes[:, :2])) < TOL
    assert err(dec(codes[:, :1].cuda()), ora.forward(codes[:, :1])) < TOL
    # an offline call leaves the state cold: the same call again gives the same audio
    a = dec(codes.cuda()).clone()
    assert err(dec(codes.cuda()), a.cpu()) == 0.0
    with dec.streaming(1):
        with pytest.raises(AssertionError):
            dec.streaming(1)


def test_small_reset_restarts_cold(small):
    d, ora, dec = small
    g = torch.Generator().manual_seed(3)
    codes = torch.randint(0, d.codebook_size, (1, d.n_codebooks, 5), generator=g).cuda()
    with dec.streaming(1):
        first = torch.cat([dec(codes[:, :, t:t + 1]).clone() for t in range(5)], dim=-1)
        dec.reset_streaming()
        again = torch.cat([dec(codes[:, :, t:t + 1]).clone() for t in range(5)], dim=-1)
    assert err(first, again.cpu()) == 0.0


def test_small_graph_replays_equal_eager(small):
    d, ora, dec = small
    g = torch.Generator().manual_seed(5)
    codes = torch.randint(0, d.codebook_size, (1, d.n_codebooks, 7), generator=g).cuda()
    with dec.streaming(1):
        eager = [dec(codes[:, :, t:t + 1]).clone() for t in range(7)]
    dec.setup_streaming_graph(1)
    try:
        with dec.streaming(1):
            for t in range(7):
                got = dec(codes[:, :, t:t + 1])
                torch.cuda.synchronize()
                assert err(got, eager[t].cpu()) == 0.0, t
    finally:
        dec._graphs.clear()


def test_persistent_trunk_equals_kernel_sequence(small):
    """The one-column steps run as one persistent kernel by default; switched off they are separate
    launches.  Same sums in another order."""
    d, ora, dec = small
    assert dec.persistent()
    g = torch.Generator().manual_seed(8)
    codes = torch.randint(0, d.codebook_size, (1, d.n_codebooks, 12), generator=g).cuda()
    a = dec(codes).clone()
    try:
        assert not dec.persistent(0)
        b = dec(codes).clone()
        assert err(a, b.cpu()) < 2e-5
        assert err(dec(codes[:, :2]), ora.forward(codes[:, :2].cpu())) < TOL
    finally:
        assert dec.persistent(1)


@pytest.mark.parametrize("nwg", [96, 128, 40])
def test_persistent_trunk_on_fewer_workgroups(small, full, nwg):
    """vui_codec_workgroups: the persistent kernel on part of the GPU (more rows of every matrix per workgroup, the
    row plan of its second instantiation) against the oracle at reduced dims and against the reference's own vectors
    at the real dims; 40 workgroups cannot hold the real model's rows and are refused there."""
    d, ora, dec = small
    g = torch.Generator().manual_seed(9)
    codes = torch.randint(0, d.codebook_size, (1, d.n_codebooks, 12), generator=g).cuda()
    try:
        dec.workgroups(nwg)
        assert dec.persistent()
        assert err(dec(codes), ora.forward(codes.cpu())) < TOL
    finally:
        dec.workgroups(256)
    df, sdf, decf, fx = full
    try:
        if nwg < 96:
            with pytest.raises(RuntimeError, match="rows per wave"):
                decf.workgroups(nwg)
            return
        decf.workgroups(nwg)
        codes = fx["codes"].cuda()
        with decf.streaming(1):
            st = torch.cat([decf(codes[:, :, t:t + 1]).clone() for t in range(codes.shape[2])], dim=-1)
        assert err(st, fx["stream"]) < TOL, err(st, fx["stream"])
    finally:
        decf.workgroups(256)


def test_errors_are_reported(small):
    d, ora, dec = small
    bad = torch.full((1, d.n_codebooks, 1), d.codebook_size, dtype=torch.long).cuda()
    with dec.streaming(1):
        dec(bad)
        with pytest.raises(RuntimeError, match="outside"):
            dec.frames_since_reset()
    with pytest.raises(ValueError):
        dec(torch.zeros(1, d.n_codebooks + 1, 1, dtype=torch.long).cuda())
    with pytest.raises(ValueError, match="window"):
        dec(torch.zeros(1, d.n_codebooks, d.max_seq + 1, dtype=torch.long).cuda())
    # a stream longer than the cache: flagged, nothing out of bounds
    with dec.streaming(1):
        z = torch.zeros(1, d.n_codebooks, 1, dtype=torch.long).cuda()
        for _ in range(d.max_seq + 1):
            dec(z)
        with pytest.raises(RuntimeError, match="max_seq"):
            dec.frames_since_reset()


def test_unsupported_dims_raise():
    from vui_amd.codec import CodecConfig, QwenCodecDecoder

    with pytest.raises(ValueError, match="multiple of 32"):
        QwenCodecDecoder({}, CodecConfig(latent_dim=24), device="cuda")


def test_full_dims_against_reference_vectors(full):
    d, sd, dec, fx = full
    codes = fx["codes"].cuda()
    with dec.streaming(1):
        st = torch.cat([dec(codes[:, :, t:t + 1]).clone() for t in range(codes.shape[2])], dim=-1)
    assert err(st, fx["stream"]) < TOL, err(st, fx["stream"])
    assert err(dec(codes), fx["offline"]) < TOL
    assert err(dec(codes[:, :8, :2]), fx["offline_q8"]) < TOL
    assert st.shape[-1] == 4 * 1920


def _digest(a):
    a = a.detach().cpu().reshape(-1).double()
    return np.array([a.sum().item(), a.abs().sum().item(), *a[:4].tolist(), *a[-4:].tolist()])


def test_full_dims_codec_ctx_session(full):
    """The reference's CodecCtx session: prompt 30 + 10 added, prefill seeds 40 frames, 90 streamed
    frames with the cold restart after 125."""
    from vui_amd.codec import CodecCtx

    d, sd, dec, fx = full
    ctx = CodecCtx(dec)
    ctx.set_prompt(fx["ctx_prompt"])
    ctx.add(fx["ctx_extra"])
    ctx.prefill()
    assert ctx._frames_since_prefill == 40
    frames = fx["ctx_frames"].cuda()
    for t in range(frames.shape[0]):
        a = ctx.decode_frame(frames[t].view(1, -1, 1))
        assert ctx._frames_since_prefill == int(fx["ctx_fsp"][t])
        got, ref = _digest(a), fx["ctx_digest"][t].numpy()
        assert abs(got[0] - ref[0]) < 0.1 and abs(got[1] - ref[1]) < 0.1, (t, got[:2], ref[:2])
        assert np.abs(got[2:] - ref[2:]).max() < 5e-4, t
    assert ctx.n_frames == 130
    ctx.reset()
    assert not dec.is_streaming
