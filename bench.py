"""Headline benchmark: Vui Nano codec frames/s at batch 1, bf16, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--preset A|B] [--no-cpu]

Workload (benchmark configuration 4, end-to-end streaming at batch 1): random-init weights
N(0, 0.02) from seed 0 in the Vui Nano architecture, a synthetic voice prefix of 512 codec
frames (uniform token ids) plus 64 uniform text tokens prefilled into the KV cache, then K
codec frames generated with the whole per-frame step (backbone step, code-0 sampling with
repetition penalty, depth head over all 16 codebooks) replayed as one HIP graph.  One
"step" is one codec frame.  Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published


def frame_bytes(m, L_avg: float, esz: int = 2) -> dict:
    """Algorithmic HBM bytes of one frame: every weight, norm vector and embedding row that must be
    read once, the KV rows read and written, for the backbone step and the depth head."""
    d, F, H, KV, hd = m.d_model, m.ffn, m.n_heads, m.kv_heads, m.head_dim
    Q, CS, R, Fr, Lr = m.n_quantizers, m.codebook_size, m.rq_d_model, m.rq_ffn, m.rq_n_layers
    layer_w = ((H + 2 * KV) * hd * d + d * d + 3 * F * d) * esz + 2 * d * esz
    kv_row = 2 * KV * hd * esz
    backbone = m.n_layers * (layer_w + kv_row * (L_avg + 1) + kv_row) + (CS * d + 2 * d + Q * d) * esz
    rq_layer = (3 * R * R + R * R + 3 * Fr * R) * esz + 2 * R * esz
    rq = Lr * rq_layer + (R * d if R != d else 0) * esz + (Q - 1) * CS * R * esz + (Q * R + Q * R + R) * esz
    return {"backbone": backbone, "rq_unique": rq, "frame": backbone + rq}


def gpu_bench(args):
    import torch

    from vui_amd.engine import Engine, GenConfig
    from vui_amd.model import Vui
    from vui_amd.synthetic import nano_for_cache, synthetic_state_dict

    torch.manual_seed(0)
    n_prefix, n_text = 512, 64
    K, W = args.steps, args.warmup
    d = nano_for_cache(args.preset, 64).model  # architecture numbers
    n_lat = min(K, 200)  # frames of the separate latency pass
    max_seq = 64 * ((n_prefix + n_text + K + W + n_lat + 2 + 63) // 64)
    t0 = time.time()
    sd = synthetic_state_dict(d, seed=0)
    model = Vui(nano_for_cache(args.preset, max_seq), sd, device="cuda", dtype=torch.bfloat16, int8=args.int8)
    eng = Engine(model=model, max_rows=1, max_seq=max_seq)
    row = eng.new_row()
    g = torch.Generator().manual_seed(0)
    prefix = torch.randint(0, d.codebook_size, (n_prefix, d.n_quantizers), generator=g).cuda()
    ids = torch.randint(0, d.vocab_size, (n_text,), generator=g).cuda()
    with torch.inference_mode():
        row.prefill_emb(model.embed_audio(prefix[None]).to(torch.bfloat16))
        h = row.prefill_emb(model.token_emb(ids[None]))[:, -1]
    torch.cuda.synchronize()
    setup_s = time.time() - t0
    cfg = GenConfig()  # temperature 0.9, top-k 100, repetition penalty 1.1 over 24 frames
    # frame 0 eagerly, then the captured frame graph
    n_total = 1 + W + K + n_lat
    eng.generate([row], h, 1, cfg)
    gr, frames, eos, _ = eng._frame_graph(1, cfg, None, n_total)
    for _ in range(W):
        gr.replay()
    torch.cuda.synchronize()
    L_start = row.offset
    # the timed region: exactly K steps between two events and two synchronisations, nothing else in the stream
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t_host0 = time.perf_counter()
    e0.record()
    for i in range(K):
        gr.replay()
    e1.record()
    torch.cuda.synchronize()
    t_host = time.perf_counter() - t_host0
    L_end = row.offset
    assert L_end - L_start == K, (L_start, L_end)
    total_ms = e0.elapsed_time(e1)
    ms_per = max(total_ms, t_host * 1e3) / K
    fps = 1e3 / ms_per
    # per-frame latency from a pass of its own (an event after every replay costs ~7 us per frame, which the timed
    # region above does not pay): the next n_lat frames of the same stream
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(n_lat + 1)]
    ev[0].record()
    for i in range(n_lat):
        gr.replay()
        ev[i + 1].record()
    torch.cuda.synchronize()
    lat = sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(n_lat))
    fb = frame_bytes(model.config.model, (L_start + L_end) / 2.0)
    if args.int8:  # the backbone's matrices are one byte per weight plus a bf16 scale per row
        mm = model.config.model
        w16 = mm.n_layers * ((mm.n_heads + 2 * mm.kv_heads) * mm.head_dim * mm.d_model + mm.d_model * mm.d_model + 3 * mm.ffn * mm.d_model) * 2
        rows_ = mm.n_layers * ((mm.n_heads + 2 * mm.kv_heads) * mm.head_dim + 2 * mm.d_model + 2 * mm.ffn)
        fb["backbone"] += -w16 // 2 + rows_ * 2
        fb["frame"] = fb["backbone"] + fb["rq_unique"]
    out = {
        "metric": "codec frames/sec at batch 1 (Vui Nano bf16)", "value": round(fps, 2), "unit": "frames/s",
        "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": round(ms_per, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "rtf": round(fps / 12.5, 2), "p50_ms": round(lat[len(lat) // 2], 4), "p99_ms": round(lat[int(len(lat) * 0.99)], 4),
        "config": {"workload": "e2e_b1: 512-frame voice prefix + 64 text tokens prefilled, then one HIP-graph "
                               "replay per codec frame (backbone step + code-0 sampling + depth head, 16 codebooks)",
                   "preset": args.preset, "backbone_weights": "int8 (weight-only, per-row bf16 scales)" if args.int8 else "bf16",
                   "kv_len": [L_start, L_end], "sampling": "T=0.9 top-k=100 rep=1.1/24",
                   "latency_sample": f"p50/p99 over the {n_lat} frames after the timed region, one event per frame",
                   "setup_s": round(setup_s, 1)},
        "frame_bytes": {k: int(v) for k, v in fb.items()},
        "fused": bool(model._native.fused(-1)),
    }
    return out, (model, eng, d, sd)


# Figures that rocprofv3 counters gave in runs of their own (a counter run serialises every dispatch, so they cannot be
# taken inside this program's timed region); every line that carries one names the file it comes from.
# HBM traffic of one frame_kernel launch (whole frame, bf16): FETCH_SIZE and WRITE_SIZE, KiB per dispatch, each scaled
# by what the same counter reads for a plain 512 MiB device copy (bench.py --calib): 2.000 and 1.000.
MEASURED_TRAFFIC = {"bytes": 488_214_606, "source": "profiles/frame_kernel_e2e_b1.txt", "cache_length": [577, 681],
                    "algorithmic_bytes_there": 415289344,
                    "command": "rocprofv3 --pmc FETCH_SIZE (then WRITE_SIZE) -- python3 bench.py --steps 50 --warmup 5 --no-cpu --no-b16 --no-sweep --calib"}
# MFMA busy cycles / busy cycles of the two persistent kernels of the 16-stream step.
MEASURED_B16_MFMA_BUSY = {"bb_batch_kernel": 0.37, "rq_batch_kernel": 0.50, "source": "profiles/e2e_b16_int8_step_kernels.txt",
                          "command": "rocprofv3 --pmc SQ_BUSY_CYCLES SQ_VALU_MFMA_BUSY_CYCLES -- python3 bench.py --b16-only --steps 2"}


def kernel_roofline(out, fb):
    """The dominant kernel is frame_kernel: one launch per codec frame holds the whole step, so its
    average duration is the timed region's HIP-event time per replay (same stream), and its
    algorithmic bytes are those of one frame at the run's mean cache length."""
    us = out["ms_per_step"] * 1e3
    ach = fb["frame"] / (us * 1e-6) / 1e9
    return {"bound": "hbm", "kernel": "frame_kernel (backbone step + code-0 sampling + depth head, one launch per frame)",
            "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBS, 4),
            "traffic": MEASURED_TRAFFIC["bytes"], "traffic_measured_at": {k: v for k, v in MEASURED_TRAFFIC.items() if k != "bytes"},
            "us_per_launch": round(us, 2), "algorithmic_bytes": int(fb["frame"])}


def vocoder_line():
    """Streaming vocoder (fp32) at the reference's dims: codes of one frame -> 1920 samples from its captured
    graph, 200 frames.  Bytes = every weight one frame must read (all but the encoder-side projections and
    the unused codebook rows)."""
    import torch

    from vui_amd.codec import CodecConfig, QwenCodecDecoder, codec_state_dict_shapes
    from vui_amd.synthetic import synthetic_codec_state_dict

    ccfg = CodecConfig()
    voc = QwenCodecDecoder(synthetic_codec_state_dict(ccfg, 0), ccfg)
    voc.setup_streaming_graph(1)
    g = torch.Generator().manual_seed(0)
    voc._stream_codes_in.copy_(torch.randint(0, ccfg.codebook_size, (ccfg.n_codebooks,), generator=g).cuda())
    shapes = codec_state_dict_shapes(ccfg)
    cb = sum(math.prod(v) for k, v in shapes.items() if not (k.startswith("quantizer") and "input_proj" in k))
    cb -= sum(math.prod(v) for k, v in shapes.items() if k.endswith("embed"))
    cb = (cb + ccfg.n_codebooks * ccfg.codebook_dim) * 4
    gr = voc._graphs[ccfg.n_codebooks]
    n = 200
    with voc.streaming(1):
        for _ in range(3):
            gr.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            gr.replay()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / n
    return voc, {"config": "vocoder_b1", "dtype": "f32", "frames": n, "us_per_frame": round(us, 1), "samples_per_frame": voc.hop,
                 "rtf": round(1e6 / us / 12.5, 1), "weight_bytes": int(cb), "achieved_GBs": round(cb / us / 1e3, 1),
                 "hbm_frac": round(cb / us / 1e3 / HBM_PEAK_GBS, 4)}


def prefill_line(model2, eng2, g, loop_too=True, reps=5, name="prefill_b1"):
    """Prompt ingestion: 576 positions (512 audio frames + 64 text tokens) in one pass per layer against the
    position-by-position path; flops = 2 x positions x backbone weights (attention is a few % more)."""
    import torch

    m = model2.config.model
    emb = (torch.randn(1, 576, m.d_model, generator=g) * 0.08).to(torch.bfloat16).cuda()
    dec = model2.decoder

    def prefill_once():
        eng2.seq_lens[0] = 0
        dec.forward_flash(emb, None)

    def timed(fn, n):
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / n

    prefill_once()
    us_pass = timed(prefill_once, reps)
    us_loop = 0.0
    if loop_too:
        dec.PREFILL_MIN = 10 ** 9
        prefill_once()
        us_loop = timed(prefill_once, 2)
        dec.PREFILL_MIN = 4
    wparams = (frame_bytes(m, 0)["backbone"] - 67584 - m.n_quantizers * m.d_model * 2 - 3145728) / 2
    fl = 2.0 * 576 * wparams
    return {"config": name, "positions": 576, "ms_one_pass": round(us_pass / 1e3, 3), "ms_position_by_position": round(us_loop / 1e3, 2),
            "achieved_TFLOPs": round(fl / us_pass / 1e6, 1), "mfma_frac": round(fl / us_pass / 1e6 / 2500.0, 4)}


def b16_line(sd, preset="A", n=100):
    """Config 5: 16 streams, int8 backbone weights, ragged caches U[128, 2048] filled N(0, 1), n frame steps
    from one captured graph (backbone kernel sequence + persistent depth head)."""
    import torch

    from vui_amd.engine import Engine, GenConfig
    from vui_amd.model import Vui
    from vui_amd.synthetic import nano_for_cache

    S = 2048 + 256
    model5 = Vui(nano_for_cache(preset, S), sd, device="cuda", dtype=torch.bfloat16, int8=True)
    m = model5.config.model
    eng5 = Engine(model=model5, max_rows=16, max_seq=S)
    model5.decoder._k.normal_()
    model5.decoder._v.normal_()
    g = torch.Generator().manual_seed(5)
    lens = torch.randint(128, 2049, (16,), generator=g)
    rows = [eng5.new_row() for _ in range(16)]
    eng5.seq_lens[:16] = lens.to(torch.int32).cuda()
    hid16 = torch.randn(16, m.d_model, generator=g).to(torch.bfloat16).cuda()
    eng5.generate(rows, hid16, 1, GenConfig())
    gr5, _, _, _ = eng5._frame_graph(16, GenConfig(), None, n + 4)
    eng5.seq_lens[:16] = lens.to(torch.int32).cuda()
    for _ in range(3):
        gr5.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(n):
        gr5.replay()
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / n
    kv_bytes = float((lens.float() + 3 + n / 2 + 1).sum()) * 2 * m.kv_heads * m.head_dim * 2 * m.n_layers
    wbytes = frame_bytes(m, 0, 1)["backbone"] - (m.n_quantizers * m.d_model + 2 * m.kv_heads * m.head_dim * 2 * m.n_layers)
    gbs = (kv_bytes + wbytes) / us / 1e3
    return {"config": "e2e_b16_int8_ragged", "us_per_frame_step": round(us, 1), "aggregate_frames_per_s": round(16e6 / us, 1),
            "rtf": round(16e6 / us / 12.5, 1), "steps": n, "kv_bytes": int(kv_bytes), "int8_weight_bytes": int(wbytes),
            "achieved_GBs": round(gbs, 1), "hbm_frac": round(gbs / HBM_PEAK_GBS, 4), "mfma_busy_frac": MEASURED_B16_MFMA_BUSY}


def phase_clock(args):
    """Wall-clock stamps that one workgroup of frame_kernel takes at its phase boundaries (vui_debug_phase_clock),
    of one frame at cache length ~630: mean and total microseconds per pair of consecutive stamp ids.  The ids
    are the TS(n) marks of frame.hip (1-6: a backbone layer; 30-: a depth-head layer pass)."""
    import collections

    import torch

    from vui_amd.engine import Engine, GenConfig
    from vui_amd.model import Vui
    from vui_amd.synthetic import nano_for_cache, synthetic_state_dict

    d = nano_for_cache(args.preset, 64).model
    S = 2304
    model = Vui(nano_for_cache(args.preset, S), synthetic_state_dict(d, seed=0), device="cuda", dtype=torch.bfloat16, int8=args.int8)
    eng = Engine(model=model, max_rows=1, max_seq=S)
    row = eng.new_row()
    model.decoder._k.normal_()
    model.decoder._v.normal_()
    eng.seq_lens[0] = 600
    g = torch.Generator().manual_seed(0)
    h = torch.randn(1, d.d_model, generator=g).to(torch.bfloat16).cuda()
    cfg = GenConfig()
    eng.generate([row], h, 30, cfg)
    cap = 1000  # stamps the kernel keeps per launch
    buf = torch.zeros(4 * (cap + 1), dtype=torch.int64, device="cuda")
    nat = model._native
    nat.lib.vui_debug_phase_clock(nat.handle, buf.data_ptr(), cap, args.phase_clock_wg)
    eng._frame_graphs = {}
    eng.generate([row], h, 4, cfg)
    torch.cuda.synchronize()
    nat.status()
    b = buf.cpu().tolist()
    n = b[cap] & 0xFFFFFFFF
    ev = [(x >> 8, x & 255) for x in b[:n]]
    seg = collections.defaultdict(list)
    for (t0, i0), (t1, i1) in zip(ev, ev[1:]):
        seg[(i0, i1)].append((t1 - t0) / 100.0)  # the clock counts 100 MHz
    print(json.dumps({"config": "frame_kernel_phase_clock", "int8": bool(args.int8), "workgroup": args.phase_clock_wg, "stamps": n,
                      "segments": [{"from": k[0], "to": k[1], "n": len(v), "mean_us": round(sum(v) / len(v), 3),
                                    "total_us": round(sum(v), 1)} for k, v in sorted(seg.items())]}))


def bb_phase_clock(args):
    """Phase stamps of one workgroup of bb_batch_kernel (a library built with -DVUI_BB_CLOCK, e.g.
    VUI_EXTRA_HIPCC_FLAGS=-DVUI_BB_CLOCK python -m vui_amd.build): B rows of benchmark configuration 5, five
    steps, the stamps of the last.  Per layer: QKV, attention pieces, merge, out_proj, W1/W3 + SwiGLU, W2."""
    import ctypes as C

    import torch

    from vui_amd.engine import Engine
    from vui_amd.model import Vui
    from vui_amd.synthetic import nano_for_cache, synthetic_state_dict

    B = args.bb_phase_clock
    d = nano_for_cache(args.preset, 64).model
    S = 2304
    model = Vui(nano_for_cache(args.preset, S), synthetic_state_dict(d, seed=0), device="cuda", dtype=torch.bfloat16, int8=args.int8)
    lib = model._native.lib
    if not hasattr(lib, "vui_debug_bb_batch_clock"):
        sys.exit("this library was built without -DVUI_BB_CLOCK")
    eng = Engine(model=model, max_rows=16, max_seq=S)
    model.decoder._k.normal_()
    model.decoder._v.normal_()
    g = torch.Generator().manual_seed(5)
    lens = torch.randint(128, 2049, (16,), generator=g).to(torch.int32)
    codes = torch.randint(0, d.codebook_size, (16, d.n_quantizers), generator=g).cuda()
    buf = torch.zeros(256, dtype=torch.int64, device="cuda")
    lib.vui_debug_bb_batch_clock.argtypes = [C.c_void_p, C.c_int]
    lib.vui_debug_bb_batch_clock(buf.data_ptr(), args.phase_clock_wg)
    st = torch.cuda.current_stream().cuda_stream
    hid = torch.empty(B, d.d_model, dtype=torch.bfloat16, device="cuda")
    cb0 = torch.empty(B, d.codebook_size, dtype=torch.bfloat16, device="cuda")
    eos = torch.empty(B, 1, dtype=torch.bfloat16, device="cuda")
    for _ in range(5):
        eng.seq_lens.zero_()
        eng.seq_lens[:B] = lens[:B].cuda()
        model.decoder._step(codes=codes[:B], emb=None, slot_idx=None, seq_inc=None, B=B, hidden_out=hid, cb0_out=cb0,
                            eos_out=eos, n_splits=8, stream=st)
    torch.cuda.synchronize()
    model._native.status()
    b = buf.cpu().tolist()
    ts = b[:b[255]]
    names = ["qkv", "attention_pieces", "merge", "out_proj", "swiglu", "w2"]  # stamps: start, six per layer, final, end
    L = d.n_layers
    per = {k: [] for k in names}
    for l in range(L):
        for k in range(6):
            per[names[k]].append((ts[1 + 6 * l + k + 1] - ts[1 + 6 * l + k]) / 100.0)
    print(json.dumps({"config": "bb_batch_kernel_phase_clock", "rows": B, "int8": bool(args.int8), "workgroup": args.phase_clock_wg,
                      "total_us": (ts[-1] - ts[0]) / 100.0, "setup_us": (ts[1] - ts[0]) / 100.0,
                      "final_us": (ts[-1] - ts[1 + 6 * L]) / 100.0,
                      "per_layer_mean_us": {k: round(sum(v) / L, 2) for k, v in per.items()}}))


def split_audio_line(sd, preset="A", split_cus=160):
    """A streamed turn with audio out on a divided GPU (Engine(split_cus=...)): decode step on split_cus compute
    units, vocoder of the previous frame beside it on the rest; 4 chunks, wall clock."""
    import torch

    from vui_amd.codec import CodecConfig, QwenCodecDecoder
    from vui_amd.engine import Chunk, Engine, GenConfig
    from vui_amd.model import Vui
    from vui_amd.synthetic import nano_for_cache, synthetic_codec_state_dict

    model = Vui(nano_for_cache(preset, 1024), sd, device="cuda", dtype=torch.bfloat16)
    ccfg = CodecConfig()
    voc = QwenCodecDecoder(synthetic_codec_state_dict(ccfg, 0), ccfg)
    eng = Engine(model=model, codec=voc, max_rows=1, max_seq=1024, split_cus=split_cus)
    g = torch.Generator().manual_seed(0)
    emb = (torch.randn(1, 16, model.config.model.d_model, generator=g) * 0.08).to(torch.bfloat16).cuda()
    chunks = [Chunk(emb=emb, n_words=40) for _ in range(4)]
    cfg_s = GenConfig(eos_threshold=2.0, max_secs=60.0)
    row = eng.new_row()
    n_out = sum(1 for _ in row.stream(chunks[:1], cfg_s))  # warm: graph captures
    row.reset()
    row._codec_ctx.reset()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    n_out, t_first = 0, 0.0
    for audio in row.stream(chunks, cfg_s):
        if n_out == 0:
            audio.cpu()  # the first frame's samples on the host
            t_first = time.perf_counter() - t0
        n_out += 1
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    model._native.status()  # raises if a persistent launch gave up a wait
    voc.frames_since_reset()  # raises if the vocoder flagged a bad code or a frame beyond its window
    return {"config": f"stream_b1_audio_split{split_cus}", "frames": n_out, "chunks": 4, "ms_per_frame_wall": round(dt * 1e3 / n_out, 4),
            "frames_per_s": round(n_out / dt, 1), "rtf": round(n_out / dt / 12.5, 2), "first_audio_ms": round(t_first * 1e3, 3),
            "vocoder_persistent_workgroups": torch.cuda.get_device_properties(0).multi_processor_count - split_cus if voc.persistent() else 0}


def rq_phase_clock(args):
    """Phase stamps of one workgroup of rq_batch_kernel at codebook 8 (a library built with -DVUI_RB_CLOCK): the
    depth head of ROWS rows, three calls, the stamps of the last.  Per layer: norm + QKV tiles, attention,
    out_proj, norm + W1/W3 + SwiGLU, W2; then the logits head and the draw."""
    import ctypes as C

    import torch

    from vui_amd.model import Vui
    from vui_amd.synthetic import nano_for_cache, synthetic_state_dict

    B = args.rq_phase_clock
    d = nano_for_cache(args.preset, 64).model
    model = Vui(nano_for_cache(args.preset, 256), synthetic_state_dict(d, seed=0), device="cuda", dtype=torch.bfloat16)
    model.decoder.allocate_flash_kv_cache(1, model.device, torch.bfloat16, max_seqlen=256)
    lib = model._native.lib
    if not hasattr(lib, "vui_debug_rq_batch_clock"):
        sys.exit("this library was built without -DVUI_RB_CLOCK")
    buf = torch.zeros(64, dtype=torch.int64, device="cuda")
    lib.vui_debug_rq_batch_clock.argtypes = [C.c_void_p, C.c_int]
    lib.vui_debug_rq_batch_clock(buf.data_ptr(), args.phase_clock_wg)
    g = torch.Generator().manual_seed(0)
    hid = torch.randn(B, d.d_model, generator=g).to(torch.bfloat16).cuda()
    c0 = torch.randint(0, d.codebook_size, (B,), generator=g).cuda()
    for _ in range(3):
        model.rq_transformer.generate(hid, c0, temperature=0.8, top_k=50)
    torch.cuda.synchronize()
    model._native.status()
    b = buf.cpu().tolist()
    ts = b[:b[63]]
    L = d.rq_n_layers
    names = ["qkv", "attention", "out_proj", "swiglu", "w2"]
    per = {k: [] for k in names}
    for l in range(L):
        for k in range(5):
            nxt = ts[5 * l + k + 1]
            per[names[k]].append((nxt - ts[5 * l + k]) / 100.0)
    print(json.dumps({"config": "rq_batch_kernel_phase_clock", "rows": B, "workgroup": args.phase_clock_wg, "codebook": 8,
                      "per_layer_mean_us": {k: round(sum(v) / L, 2) for k, v in per.items()},
                      "layers_us": round((ts[5 * L] - ts[0]) / 100.0, 2), "logits_and_draw_us": round((ts[-1] - ts[5 * L]) / 100.0, 2)}))


def batch_sweep(sd, preset="A", n=40, batches=(1, 2, 4, 8, 16)):
    """The frame step (backbone step + code-0 draw + depth head, one captured graph per batch size) for 1..16
    concurrent streams, with bf16 and with int8 backbone weights: ragged caches as in benchmark configuration 5
    (lengths U[128, 2048] from seed 5, the first B of them; filled N(0, 1)), n replays each after 3 warm-ups."""
    import torch

    from vui_amd.engine import Engine, GenConfig
    from vui_amd.model import Vui
    from vui_amd.synthetic import nano_for_cache

    S = 2048 + 256
    g = torch.Generator().manual_seed(5)
    lens = torch.randint(128, 2049, (16,), generator=g).to(torch.int32)
    out = []
    for int8 in (False, True):
        model = Vui(nano_for_cache(preset, S), sd, device="cuda", dtype=torch.bfloat16, int8=int8)
        m = model.config.model
        eng = Engine(model=model, max_rows=16, max_seq=S)
        model.decoder._k.normal_()
        model.decoder._v.normal_()
        rows = [eng.new_row() for _ in range(16)]
        hid = torch.randn(16, m.d_model, generator=g).to(torch.bfloat16).cuda()
        for B in batches:
            eng.seq_lens.zero_()
            eng.seq_lens[:B] = lens[:B].cuda()
            eng.generate(rows[:B], hid[:B], 1, GenConfig())
            gr, _, _, _ = eng._frame_graph(B, GenConfig(), None, n + 4)
            eng.seq_lens[:B] = lens[:B].cuda()
            for _ in range(3):
                gr.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(n):
                gr.replay()
            e1.record()
            torch.cuda.synchronize()
            model._native.status()
            us = e0.elapsed_time(e1) * 1e3 / n
            out.append({"B": B, "weights": "int8" if int8 else "bf16", "us_per_step": round(us, 1),
                        "aggregate_frames_per_s": round(B * 1e6 / us, 1)})
        del eng, model, rows
        torch.cuda.empty_cache()
    return out


def serve_line(sd, preset="A", n_requests=32, max_rows=16, int8=False):
    """Continuous batching as a served workload (Engine.render_continuous): n_requests requests, each a
    256-position prompt and two text chunks of 16 positions / 5 words, through max_rows rows (bf16); EOS off,
    so every chunk runs to its 40-frame cap.  Wall clock includes prompt ingestion, the host loop, the
    per-step EOS read and the refills."""
    import torch

    from vui_amd.engine import Chunk, Engine, GenConfig, RenderRequest
    from vui_amd.model import Vui
    from vui_amd.synthetic import nano_for_cache

    S = 512
    model = Vui(nano_for_cache(preset, S), sd, device="cuda", dtype=torch.bfloat16, int8=int8)
    m = model.config.model
    eng = Engine(model=model, max_rows=max_rows, max_seq=S)
    g = torch.Generator().manual_seed(9)

    def emb(n):
        return (torch.randn(1, n, m.d_model, generator=g) * 0.08).to(torch.bfloat16).cuda()

    reqs = [RenderRequest(chunks=[Chunk(emb=emb(16), n_words=5) for _ in range(2)], prompt_emb=emb(256)) for _ in range(n_requests)]
    cfg = GenConfig(eos_threshold=2.0)
    eng.render_continuous(reqs[:max_rows + 1], cfg)  # warm: graph capture for every bucket on the way down
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    out = eng.render_continuous(reqs, cfg)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    n_frames = sum(len(o) for o in out)
    return {"config": "continuous_batching_b16" + ("_int8" if int8 else ""), "requests": n_requests, "rows": max_rows, "frames": n_frames,
            "wall_s": round(dt, 3), "aggregate_frames_per_s": round(n_frames / dt, 1), "rtf_aggregate": round(n_frames / dt / 12.5, 1)}


def copy_line():
    """The practical bandwidth ceiling of the box: a plain 1 GiB device-to-device copy (reads + writes)."""
    import torch

    src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").random_(0, 255)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(10):
        dst.copy_(src)
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / 10
    return {"config": "device_copy_1GiB", "us": round(us, 1), "read_plus_write_GBs": round(2 * (1 << 30) / us / 1e3, 1),
            "frac_of_8TBs": round(2 * (1 << 30) / us / 1e3 / HBM_PEAK_GBS, 3)}


def suite(model, eng, d, sd, preset="A"):
    """Extra lines for the other benchmark configs: backbone step at KV 256/1024/4096, depth head alone,
    16 int8 streams with ragged caches."""
    import torch

    from vui_amd.engine import Engine, GenConfig
    from vui_amd.model import Vui
    from vui_amd.synthetic import nano_for_cache

    lines = []
    m = model.config.model

    def timed(fn, n):
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / n

    # config 2: backbone decode step, B=1, N(0,1) cache at three lengths (the walk over 200 steps is centred on L)
    model2 = Vui(nano_for_cache(preset, 4608), sd, device="cuda", dtype=torch.bfloat16)
    eng2 = Engine(model=model2, max_rows=1, max_seq=4608)
    model2.decoder._k.normal_()
    model2.decoder._v.normal_()
    eng2._decode_step()
    for L in (256, 1024, 4096):
        n = 200
        eng2.seq_lens[0] = L - n // 2
        us = timed(eng2._decode_graph.replay, n)
        b = frame_bytes(m, L)["backbone"]
        lines.append({"config": "backbone_step_b1", "kv_len": L, "us_per_step": round(us, 2), "us_per_layer": round(us / m.n_layers, 2),
                      "algorithmic_bytes": int(b), "achieved_GBs": round(b / us / 1e3, 1), "hbm_frac": round(b / us / 1e3 / HBM_PEAK_GBS, 4)})
    # the same step with cold caches: three copies of the weights (3 x 311 MB, more than the 256 MB memory-side cache)
    # with a cache each, taken in turn, so that no step finds its weights or keys where the previous step left them
    cold = [(model2, eng2)]
    for _ in range(2):
        sdc = {k: v.clone() for k, v in sd.items()}
        mc = Vui(nano_for_cache(preset, 4608), sdc, device="cuda", dtype=torch.bfloat16)
        ec = Engine(model=mc, max_rows=1, max_seq=4608)
        mc.decoder._k.normal_()
        mc.decoder._v.normal_()
        ec._decode_step()
        cold.append((mc, ec))
    for L in (256, 1024, 4096):
        n = 198
        for _, e in cold:
            e.seq_lens[0] = L - n // 6
        k = [0]

        def step():
            cold[k[0] % 3][1]._decode_graph.replay()
            k[0] += 1

        us = timed(step, n)
        b = frame_bytes(m, L)["backbone"]
        lines.append({"config": "backbone_step_b1_cold", "kv_len": L, "weight_copies": 3, "us_per_step": round(us, 2),
                      "us_per_layer": round(us / m.n_layers, 2), "algorithmic_bytes": int(b), "achieved_GBs": round(b / us / 1e3, 1),
                      "hbm_frac": round(b / us / 1e3 / HBM_PEAK_GBS, 4)})
    for mc, ec in cold[1:]:
        mc._native.status()
    del cold, mc, ec, sdc
    # config 3: depth head alone, 1000 frames, T=0.8 top-k 50
    rq = model2.rq_transformer
    rq.setup_cuda_graph_kv(model2.device, torch.bfloat16, top_k=50, batch_sizes=(1,))
    g = torch.Generator().manual_seed(0)
    hid = torch.randn(1, m.d_model, generator=g).to(torch.bfloat16).cuda()
    c0 = torch.randint(0, m.codebook_size, (1,), generator=g).cuda()
    rq.generate_cuda_graph_kv(hid, c0, 0.8)
    gr = rq._gkv_graphs[(1, m.n_quantizers)]
    us = timed(gr.replay, 1000)
    b = frame_bytes(m, 0)["rq_unique"]
    lines.append({"config": "rq_head_b1", "frames": 1000, "us_per_frame": round(us, 2), "unique_bytes": int(b),
                  "achieved_GBs": round(b / us / 1e3, 1), "hbm_frac": round(b / us / 1e3 / HBM_PEAK_GBS, 4)})
    lines.append(prefill_line(model2, eng2, g))
    model8 = Vui(nano_for_cache(preset, 1024), sd, device="cuda", dtype=torch.bfloat16, int8=True)
    eng8 = Engine(model=model8, max_rows=1, max_seq=1024)
    lines.append(prefill_line(model8, eng8, g, name="prefill_b1_int8"))
    del model8, eng8
    emb = (torch.randn(1, 576, m.d_model, generator=g) * 0.08).to(torch.bfloat16).cuda()
    # a streamed turn: one graph replay per frame plus the host's per-frame EOS read (Row.stream)
    from vui_amd.engine import Chunk
    eng2.seq_lens[0] = 0
    row2 = eng2.new_row()
    chunks = [Chunk(emb=emb[:, :16].contiguous(), n_words=40) for _ in range(4)]
    cfg_s = GenConfig(eos_threshold=2.0, max_secs=60.0)
    n_out = sum(1 for _ in row2.stream(chunks[:1], cfg_s))  # warm: graph capture
    row2.reset()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    n_out = sum(1 for _ in row2.stream(chunks, cfg_s))
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    lines.append({"config": "stream_b1", "frames": n_out, "chunks": 4, "ms_per_frame_wall": round(dt * 1e3 / n_out, 4),
                  "frames_per_s": round(n_out / dt, 1), "rtf": round(n_out / dt / 12.5, 2)})
    # streaming vocoder, then a streamed turn with audio out (decode step + vocoder per frame, codes stay on
    # the device)
    voc, line = vocoder_line()
    lines.append(line)
    eng2.codec = voc
    eng2.seq_lens[0] = 0
    row3 = row2
    from vui_amd.codec import CodecCtx
    row3._codec_ctx = CodecCtx(voc)
    row3.reset()
    n_out = sum(1 for _ in row3.stream_audio(chunks[:1], cfg_s))
    row3.reset()
    row3._codec_ctx.reset()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    n_out, t_first = 0, 0.0
    for audio in row3.stream_audio(chunks, cfg_s):
        if n_out == 0:
            audio.cpu()  # time to the first frame's samples on the host: text of the chunk ingested, frame 0, vocoder
            t_first = time.perf_counter() - t0
        n_out += 1
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    lines.append({"config": "stream_b1_audio", "frames": n_out, "chunks": 4, "ms_per_frame_wall": round(dt * 1e3 / n_out, 4),
                  "frames_per_s": round(n_out / dt, 1), "rtf": round(n_out / dt / 12.5, 2), "first_audio_ms": round(t_first * 1e3, 3)})
    # the same turn with the GPU divided: decode step on 160 compute units, vocoder of the previous frame beside it
    # on the other 96 (Engine(split_cus=160))
    row3._codec_ctx.reset()  # closes the vocoder's open stream
    del eng2, row2, row3, model2, voc
    lines.append(split_audio_line(sd, preset))
    lines.append(b16_line(sd, preset))
    lines.append(serve_line(sd, preset))
    lines.append(serve_line(sd, preset, int8=True))
    lines.append(copy_line())
    return lines


def cpu_baseline(preset, n_frames: int = 40, n_frames_bf16: int = 16, n_prefix: int = 512, n_text: int = 64):
    """The CPU oracle (a port of the reference's CPU path) on a bounded sample of the same workload, on this
    box's host cores: the headline context (512 prefix frames through the audio embedding + 64 text ids, seed 0)
    is ingested once, then n_frames frames (backbone step + depth head, greedy as the baseline plan asks) are
    timed three times after one warm-up and the median is reported; the same in the oracle's bf16 regime on a
    shorter sample.  Threads: the box's CPU share (OMP_NUM_THREADS where the box sets it, else every CPU)."""
    import platform

    import torch

    from oracle import vui_oracle as O

    host_cpus = os.cpu_count() or 1
    threads = int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or host_cpus
    threads = max(1, min(threads, host_cpus))
    torch.set_num_threads(threads)
    d = O.Dims() if preset == "A" else O.Dims(rq_d_model=768, rq_n_layers=5, rq_n_heads=8, vocab_size=50534)
    sd = O.synthetic_state_dict(d, seed=0)
    g = torch.Generator().manual_seed(0)
    prefix = torch.randint(0, d.codebook_size, (n_prefix, d.n_quantizers), generator=g)
    ids = torch.randint(0, d.vocab_size, (n_text,), generator=g)
    cpu_model = ""
    try:
        with open("/proc/cpuinfo") as f:
            for ln in f:
                if ln.startswith("model name"):
                    cpu_model = ln.split(":", 1)[1].strip()
                    break
    except OSError:
        cpu_model = platform.processor()

    def run(dt, n):
        o = O.OracleModel(d, sd, dt, max_seqlen=n_prefix + n_text + n + 8)
        with torch.inference_mode():
            ctx = torch.cat([o.embed_audio(prefix), o.embed_text(ids)], 0)
            h = o.prefill(ctx)[-1:]
            L0 = int(o.seq_lens[0])
            times = []
            for rep in range(4):  # one warm-up, then three timed passes from the same cache state
                o.seq_lens[0] = L0
                t0 = time.perf_counter()
                o.generate_frames(h, n, temperature=1.0, top_k=1)
                times.append(time.perf_counter() - t0)
        return n / sorted(times[1:])[1]

    f32 = run(torch.float32, n_frames)
    bf16 = run(torch.bfloat16, n_frames_bf16)
    return {"value": round(f32, 3), "unit": "frames/s", "cores": threads, "kind": "port",
            "value_bf16_regime": round(bf16, 3), "rtf": round(f32 / 12.5, 3), "ms_per_frame": round(1e3 / f32, 2),
            "host_cpus": host_cpus, "cpu_model": cpu_model,
            "sample": f"fp32 oracle: {n_prefix} prefix frames + {n_text} text ids ingested, then {n_frames} greedy frames "
                      f"(backbone step + depth head), median of 3 after 1 warm-up; bf16 regime: {n_frames_bf16} frames; "
                      f"torch CPU ops, {threads} threads of {host_cpus} CPUs"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=750)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--preset", default="A", choices=["A", "B"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--int8", action="store_true", help="batch 1 with the backbone's matrices as weight-only int8")
    ap.add_argument("--no-sweep", action="store_true", help="skip the batch sweep of the default line")
    ap.add_argument("--sweep-only", action="store_true", help="print only the batch sweep (B = 1..16, bf16 and int8 weights)")
    ap.add_argument("--no-roofline", action="store_true")
    ap.add_argument("--no-b16", action="store_true", help="skip the 16-stream int8 leg of the default line")
    ap.add_argument("--suite", action="store_true", help="also print one JSON line per further benchmark config")
    ap.add_argument("--calib", action="store_true",
                    help="end with three plain 512 MiB device copies (reference points for hardware counters)")
    ap.add_argument("--prefill-only", action="store_true",
                    help="print only the prompt-ingestion line, one-pass path only (the run its rocprofv3 summary comes from)")
    ap.add_argument("--b16-only", action="store_true",
                    help="print only the 16-stream int8 line (the run its rocprofv3 summaries come from)")
    ap.add_argument("--serve-only", action="store_true",
                    help="print only the continuous-batching line (32 requests through 16 rows, wall clock)")
    ap.add_argument("--vocoder-only", action="store_true",
                    help="print only the vocoder line (the run rocprofv3 summaries of the vocoder kernels come from)")
    ap.add_argument("--split-audio-only", action="store_true",
                    help="print only the streamed turn with audio on a divided GPU (the run its rocprofv3 summary comes from)")
    ap.add_argument("--phase-clock", action="store_true",
                    help="print the phase stamps of one workgroup of the batch-1 frame kernel (with --int8: int8 weights)")
    ap.add_argument("--bb-phase-clock", type=int, default=0, metavar="ROWS",
                    help="print the phase stamps of the batched backbone kernel for ROWS rows (needs a -DVUI_BB_CLOCK build)")
    ap.add_argument("--rq-phase-clock", type=int, default=0, metavar="ROWS",
                    help="print the phase stamps of the batched depth-head kernel for ROWS rows (needs a -DVUI_RB_CLOCK build)")
    ap.add_argument("--phase-clock-wg", type=int, default=0, help="the workgroup whose stamps are taken")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU part (streams are independent); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if args.phase_clock:
        return phase_clock(args)
    if args.bb_phase_clock:
        return bb_phase_clock(args)
    if args.rq_phase_clock:
        return rq_phase_clock(args)
    if args.vocoder_only:
        print(json.dumps(vocoder_line()[1]))
        return
    if args.split_audio_only:
        from vui_amd.synthetic import nano_for_cache, synthetic_state_dict

        print(json.dumps(split_audio_line(synthetic_state_dict(nano_for_cache(args.preset, 64).model, seed=0), args.preset)))
        return
    if args.prefill_only:
        import torch

        from vui_amd.engine import Engine
        from vui_amd.model import Vui
        from vui_amd.synthetic import nano_for_cache, synthetic_state_dict

        sd = synthetic_state_dict(nano_for_cache(args.preset, 64).model, seed=0)
        model2 = Vui(nano_for_cache(args.preset, 1024), sd, device="cuda", dtype=torch.bfloat16, int8=args.int8)
        eng2 = Engine(model=model2, max_rows=1, max_seq=1024)
        print(json.dumps(prefill_line(model2, eng2, torch.Generator().manual_seed(0), loop_too=False, reps=20,
                                      name="prefill_b1_int8" if args.int8 else "prefill_b1")))
        return
    if args.serve_only:
        from vui_amd.synthetic import nano_for_cache, synthetic_state_dict

        print(json.dumps(serve_line(synthetic_state_dict(nano_for_cache(args.preset, 64).model, seed=0), args.preset, int8=args.int8)))
        return
    if args.sweep_only:
        from vui_amd.synthetic import nano_for_cache, synthetic_state_dict

        print(json.dumps({"batch_sweep": batch_sweep(synthetic_state_dict(nano_for_cache(args.preset, 64).model, seed=0), args.preset)}))
        return
    if args.b16_only:
        from vui_amd.synthetic import nano_for_cache, synthetic_state_dict

        n = args.steps if args.steps != 750 else 100  # --steps shortens the run for counter collection
        print(json.dumps(b16_line(synthetic_state_dict(nano_for_cache(args.preset, 64).model, seed=0), args.preset, n)))
        return
    out, (model, eng, d, sd) = gpu_bench(args)
    if not args.no_roofline:
        out["roofline"] = kernel_roofline(out, out["frame_bytes"])
        if args.int8 or args.preset != "A":  # the counters were read for preset A with bf16 weights only
            out["roofline"]["traffic"] = None
            out["roofline"].pop("traffic_measured_at", None)
    if not args.no_b16 and not args.suite:
        # batch 16 (benchmark configuration 5) beside the batch-1 figure, after its timed region: 16 int8 streams
        # with ragged caches, a bounded number of replays of the captured step
        out["b16"] = b16_line(sd, args.preset, n=60)
    if not args.no_sweep and not args.suite:
        del model, eng
        out["batch_sweep"] = batch_sweep(sd, args.preset)
    extra = suite(model, eng, d, sd, args.preset) if args.suite else []
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(args.preset)
    if args.calib:
        import torch

        src = torch.empty(512 << 20, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
    print(json.dumps(out))
    for ln in extra:
        print(json.dumps(ln))


if __name__ == "__main__":
    main()
