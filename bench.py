"""Benchmark of the NF4 linear-layer hot path on one MI355X.

``python bench.py --gpus 1 --steps K --warmup W`` prints ONE JSON line.

Primary workload (``metric``/``value``): a step is one launch of the decode GEMV
over the headline layer (x [1,5120] bf16 times W [13824,5120], NF4 group-64) on
weights that rotate through > 512 MB of distinct copies, so neither L2 nor the
256 MB Infinity Cache can serve them.  ``value`` is the achieved algorithmic
bandwidth in GB/s (packed codes + scales + x + y per launch), inputs resident in
HBM.  Launches are replayed from one HIP graph and timed with events on the
launch stream, so ``ms_per_step`` is the kernel's own average duration.

Extra objects on the same line:
  roofline      algorithmic bytes / average launch duration, against 8 TB/s
  cpu_baseline  the oracle's two-pass CPU linear (decode, then fp32 matmul)
                timed on this box's host cores on a bounded number of passes
  decode        resident greedy decode of the 14B-shaped model: tokens/s from
                graph replays and its fraction of the bandwidth roofline
  prefill       MFMA GEMM chunks at the 14B linear shapes, N in {8, 16, 32}
  layer_launches  the five launches of one 14B decode layer, each on its own
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# HBM bytes one GEMV launch of the primary workload moves, from FETCH_SIZE + WRITE_SIZE
# hardware counters scaled by a plain device copy (profiles/gemv_ring_rows_13824x5120_pmc.txt
# has the runs and the arithmetic).  Hardware counters cannot be read inside this process.
GEMV_TRAFFIC_BYTES = 39_428_626
MFMA_BF16_PEAK_TFLOPS = 2500.0

M, K = 13824, 5120  # headline layer: 14B gate/up projection


def algorithmic_bytes(m: int, k: int, n: int = 1) -> int:
    """Packed codes + fp16 scales + bf16 x + bf16 y for one linear."""
    kp = 64 * ((k + 63) // 64)
    return m * kp // 2 + m * (kp // 64) * 2 + 2 * k * n + 2 * m * n


def make_weights(torch, nf4, m: int, k: int, copies: int, seed: int):
    """W ~ N(0, 0.02) quantised on the GPU by the library's encoder; copies are
    independent draws so no two share bytes."""
    out = []
    g = torch.Generator(device="cuda")
    for i in range(copies):
        g.manual_seed(seed + i)
        w = torch.randn((m, k), generator=g, device="cuda", dtype=torch.float32) * 0.02
        out.append(nf4.nf4_quantize(w))
        del w
    return out


#: a timed window holds at least this many launches (a graph of fewer is replayed back to back)
MIN_WINDOW_LAUNCHES = 200


def graph_time(torch, launch, n_launches: int, reps: int = 5, min_window: int = MIN_WINDOW_LAUNCHES) -> float:
    """Capture a window of calls of ``launch(i)`` into a HIP graph, once per timed window with
    ``i`` running on from where the window before stopped (so a window never starts on the
    copies the one before it has just left in the caches), and return the median over the
    ``reps`` windows of the average milliseconds per launch.  A window is the ``n_launches``
    sequence repeated until it holds at least ``min_window`` launches (a window of a few
    launches is mostly its own start and end), all inside one graph: replaying a short graph
    back to back instead puts the gap between two graph launches, ~10 us, into every
    ``n_launches`` (9.8 against 9.2 us per launch at 20); events on the capture stream bracket
    the replay."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    repeats = max(1, -(-min_window // n_launches))
    window = n_launches * repeats
    with torch.cuda.stream(side):
        for i in range(min(n_launches, 32)):
            launch(i)
        side.synchronize()
        graphs = []
        for r in range(reps + 1):
            graph = torch.cuda.CUDAGraph()
            graph.capture_begin()
            for i in range(window):
                launch(r * window + i)
            graph.capture_end()
            graphs.append(graph)
        graphs[0].replay()   # untimed: first replay of a graph pays its upload
        for graph in graphs[1:]:
            graph.replay()
        side.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        # untimed: a card that has been idle runs its first milliseconds at a lower clock; replay
        # until two windows in a row agree to 2% (at most 0.3 s)
        t_spin = time.perf_counter()
        last = None
        while time.perf_counter() - t_spin < 0.3:
            e0.record(side)
            graphs[0].replay()
            e1.record(side)
            side.synchronize()
            now = e0.elapsed_time(e1)
            if last is not None and abs(now - last) <= 0.02 * last:
                break
            last = now
        times = []
        for graph in graphs[1:]:
            e0.record(side)
            graph.replay()
            e1.record(side)
            side.synchronize()
            times.append(e0.elapsed_time(e1))
    torch.cuda.current_stream().wait_stream(side)
    times.sort()
    return times[len(times) // 2] / window


#: kernel forms of the N=1 path, by the environment switches the library reads per launch
GEMV_FORMS = {
    # levels rounded to binary16 (11 significant bits) against x staged as binary16 times a power
    # of two (exact for bf16 x), exact products, fp32 accumulation: the default
    "f16_levels": {"CHR_NF4_GEMV_STAGED": None, "CHR_NF4_GEMV_TERMS": None},
    # levels as head + tail bf16 (17 significant bits): 8-byte lookups
    "two_term": {"CHR_NF4_GEMV_STAGED": None, "CHR_NF4_GEMV_TERMS": "2"},
    # levels rounded to one bf16
    "one_term": {"CHR_NF4_GEMV_STAGED": None, "CHR_NF4_GEMV_TERMS": "1"},
    # 16 fp32 levels, x widened to fp32, 128-bit loads (the plain kernel)
    "fp32_levels": {"CHR_NF4_GEMV_STAGED": "0", "CHR_NF4_GEMV_TERMS": None},
}


class gemv_form:
    """Select a kernel form for the launches (and captures) inside the block."""

    def __init__(self, name: str) -> None:
        self.env = GEMV_FORMS[name]
        self.saved: dict[str, str | None] = {}

    def __enter__(self):
        for k, v in self.env.items():
            self.saved[k] = os.environ.get(k)
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
        return self

    def __exit__(self, *exc):
        for k, v in self.saved.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
        return False


def bench_gemv(torch, nf4, steps: int, warmup: int, copies: int):
    by = algorithmic_bytes(M, K)
    copies = max(copies, -(-512 * 1024 * 1024 // by) + 1)
    weights = make_weights(torch, nf4, M, K, copies, seed=1234)
    g = torch.Generator(device="cuda")
    g.manual_seed(99)
    x = torch.randn(K, generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    y = torch.empty(M, dtype=torch.bfloat16, device="cuda")

    def launch(i):
        p, s = weights[i % copies]
        nf4.nf4_gemv(p, s, x, M, K, K, y)

    # eager loop: W warm-up steps, then exactly K steps between two syncs
    for i in range(warmup):
        launch(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        launch(i)
    torch.cuda.synchronize()
    eager_ms = (time.perf_counter() - t0) * 1e3 / steps
    ms = graph_time(torch, launch, steps)
    forms = {}
    for name in ("two_term", "one_term", "fp32_levels"):
        with gemv_form(name):
            forms[name] = graph_time(torch, launch, steps)
    del weights
    torch.cuda.empty_cache()
    return ms, eager_ms, copies, by, forms


def bench_gemv_shapes(torch, nf4):
    """The GEMV at the other 14B layer shapes and at the vocabulary projection: the fixed
    cost of a launch weighs less the longer the weight stream is.  Same method as the
    primary workload (graph replay, rotating copies beyond the 256 MB Infinity Cache)."""
    rows = []
    for name, m, k in (("qkv", 7168, 5120), ("o", 5120, 5120), ("down", 5120, 13824),
                       ("gate+up rows", 27648, 5120), ("lm_head", 152064, 5120)):
        by = algorithmic_bytes(m, k)
        copies = max(2, -(-600 * 1024 * 1024 // by) + 1)
        weights = make_weights(torch, nf4, m, k, copies, seed=4321)
        g = torch.Generator(device="cuda")
        g.manual_seed(98)
        x = torch.randn(k, generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
        y = torch.empty(m, dtype=torch.bfloat16, device="cuda")

        def launch(i, weights=weights, copies=copies, x=x, y=y, m=m, k=k):
            p, s = weights[i % copies]
            nf4.nf4_gemv(p, s, x, m, k, k, y)

        ms = graph_time(torch, launch, 120)
        rows.append({"layer": name, "M": m, "K": k, "us": ms * 1e3, "gbps": by / ms / 1e6,
                     "hbm_frac": by / ms / 1e6 / HBM_PEAK_GBPS})
        del weights
        torch.cuda.empty_cache()
    return rows


def bench_layer_launches(torch, nf4, contexts=(640, 2047)):
    """The five launches of one 14B-architecture decode layer, each on its own (graph replays,
    rotating weights and caches): q/k/v with the folded RMSNorm and biases, the attention at the
    given cache lengths, the o projection that merges the attention's states and adds the
    residual, gate/up with the folded RMSNorm and SwiGLU, down with the residual.  As in the
    step, the two launches that write the residual stream leave its sum of squares and the two
    that normalise it take it from there."""
    from deepfold_amd.decodev2.rope import rope_tables_torch

    k5, ffn, n_q, n_kv, hd, max_seq = 5120, 13824, 40, 8, 128, 2048
    rows = []
    dev = "cuda"
    x = torch.randn(k5, device=dev).to(torch.bfloat16)
    g = (1 + 0.05 * torch.randn(k5, device=dev)).to(torch.bfloat16)
    res = torch.randn(k5, device=dev).to(torch.bfloat16)
    parts = torch.zeros(nf4.dv2_sumsq_parts(), dtype=torch.float32, device=dev)
    parts[0] = float((x.float() ** 2).sum())

    def add(name, launch, nbytes, n=120):
        ms = graph_time(torch, launch, n)
        rows.append({"launch": name, "us": ms * 1e3, "bytes": nbytes, "gbps": nbytes / ms / 1e6,
                     "hbm_frac": nbytes / ms / 1e6 / HBM_PEAK_GBPS})

    c = 24
    q = make_weights(torch, nf4, n_q * hd, k5, c, 1)
    kk = make_weights(torch, nf4, n_kv * hd, k5, c, 2)
    v = make_weights(torch, nf4, n_kv * hd, k5, c, 3)
    yq = torch.empty(n_q * hd, dtype=torch.bfloat16, device=dev)
    yk = torch.empty(n_kv * hd, dtype=torch.bfloat16, device=dev)
    yv = torch.empty(n_kv * hd, dtype=torch.bfloat16, device=dev)
    bq, bk, bv = (torch.randn(t.numel(), device=dev).to(torch.bfloat16) for t in (yq, yk, yv))

    def qkv(i):
        j = i % c
        nf4.nf4_qkv(q[j][0], q[j][1], kk[j][0], kk[j][1], v[j][0], v[j][1], x, n_q * hd, n_kv * hd, n_kv * hd,
                    k5, k5, yq, yk, yv, bq, bk, bv, rms_w=g, sumsq_in=parts)

    add("q/k/v 7168x5120 + RMSNorm + biases", qkv, algorithmic_bytes((n_q + 2 * n_kv) * hd, k5))
    del q, kk, v
    torch.cuda.empty_cache()

    layers = 48
    kc = torch.randn(layers, max_seq, n_kv, hd, device=dev).to(torch.bfloat16)
    vc = torch.randn(layers, max_seq, n_kv, hd, device=dev).to(torch.bfloat16)
    qa = torch.randn(n_q, hd, device=dev).to(torch.bfloat16)
    ka = torch.randn(n_kv, hd, device=dev).to(torch.bfloat16)
    va = torch.randn(n_kv, hd, device=dev).to(torch.bfloat16)
    cos, sin = rope_tables_torch(max_seq, hd, 1e6, device=dev, dtype=torch.bfloat16)
    state = torch.zeros(nf4.dv2_attn_state_floats(n_q, hd), dtype=torch.float32, device=dev)
    for ctx in contexts:
        vl = torch.full((), ctx, dtype=torch.int32, device=dev)
        pos = torch.full((), ctx, dtype=torch.int64, device=dev)

        def attn(i, vl=vl, pos=pos):
            layer = i % layers
            nf4.dv2_attn_parts(qa, kc[layer], vc[layer], vl, hd ** -0.5, state, k_act=ka, v_act=va, cos=cos,
                               sin=sin, position=pos)

        add(f"attention, {ctx} cache rows (RoPE, cache write, states for the o projection)", attn,
            2 * ctx * n_kv * hd * 2, n=96)
    del kc, vc
    torch.cuda.empty_cache()

    o = make_weights(torch, nf4, k5, k5, 40, 5)
    yo = torch.empty(k5, dtype=torch.bfloat16, device=dev)
    st = torch.randn(nf4.dv2_attn_state_floats(n_q, hd), device=dev).abs()
    parts_out = torch.zeros_like(parts)
    add("o 5120x5120 + attention merge + residual",
        lambda i: nf4.dv2_gemv_attn(o[i % 40][0], o[i % 40][1], st, n_q, hd, k5, k5, k5, yo, res,
                                    sumsq_out=parts_out),
        algorithmic_bytes(k5, k5) + st.numel() * 4)
    del o
    torch.cuda.empty_cache()

    ga = make_weights(torch, nf4, ffn, k5, 10, 6)
    up = make_weights(torch, nf4, ffn, k5, 10, 7)
    ys = torch.empty(ffn, dtype=torch.bfloat16, device=dev)
    add("gate/up 2 x 13824x5120 + RMSNorm + SwiGLU",
        lambda i: nf4.nf4_swiglu(ga[i % 10][0], ga[i % 10][1], up[i % 10][0], up[i % 10][1], x, ffn, k5, k5, ys,
                                 rms_w=g, sumsq_in=parts),
        2 * algorithmic_bytes(ffn, k5) - 2 * k5 - 2 * ffn)
    del ga, up
    torch.cuda.empty_cache()

    d = make_weights(torch, nf4, k5, ffn, 18, 8)
    xd = torch.randn(ffn, device=dev).to(torch.bfloat16)
    add("down 5120x13824 + residual",
        lambda i: nf4.nf4_gemv(d[i % 18][0], d[i % 18][1], xd, k5, ffn, ffn, yo, res, sumsq_out=parts_out),
        algorithmic_bytes(k5, ffn) + 2 * k5)
    del d
    torch.cuda.empty_cache()
    return rows


def bench_prefill(torch, nf4, only=None, widths=(8, 16, 32, 64)):
    """MFMA GEMM chunks at the 14B linear shapes; weights rotate through > 512 MB.  A launch
    is the tile kernel and, where it splits K, its reduce."""
    shapes = {"qkv": (7168, 5120), "o": (5120, 5120), "gate_up": (13824, 5120), "down": (5120, 13824)}
    rows = []
    for name, (m, k) in shapes.items():
        if only and name not in only:
            continue
        by1 = algorithmic_bytes(m, k, 1)
        copies = -(-512 * 1024 * 1024 // by1) + 1
        weights = make_weights(torch, nf4, m, k, copies, seed=4321)
        for n in widths:  # 64: the chunk width of the feature-major prefill
            x = (torch.randn((k, n), device="cuda") ).to(torch.bfloat16)

            def launch(i):
                p, s = weights[i % copies]
                nf4.nf4_gemm(p, s, x, m, k, k, max_n=64)

            ms = graph_time(torch, launch, 3 * copies, reps=3)
            by = algorithmic_bytes(m, k, n)
            plan = nf4.nf4_plan(m, k, n)
            if plan["bm"] in (32, 64):
                tile = (f"stream ({plan['bm']} rows x all of K, no split)" if plan["grid_y"] == 1 else
                        f"stream ({plan['bm']} rows, K over {plan['grid_y']} workgroups that meet in the tile)")
            else:
                tile = f"split-K x{plan['grid_y']} + reduce"
            rows.append({"layer": name, "M": m, "K": k, "N": n, "us": ms * 1e3, "tile": tile,
                         "gbps": by / (ms * 1e-3) / 1e9,
                         "hbm_frac": by / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                         "mfma_frac": 2.0 * m * k * n / (ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS})
        del weights
        torch.cuda.empty_cache()
    return rows


#: the decode configurations the metric names, per architecture: (prompt tokens, prefill chunk
#: width or None for the launches' own 64, new tokens).  3B: 512-token prompt, 256 tokens.
#: 20B: 1024-token prompt prefilled in 32-position chunks, 256 tokens.  32B: the step at a
#: 2048-token context (the last 256 positions of the cache).
DECODE_CONFIGS = {
    "3b": (512, None, 256),
    "14b": (512, None, 256),
    "20b": (1024, 32, 256),
    "32b": (2048 - 256 - 1, None, 256),
}


def bench_decode(torch, spec_name: str, prompt_len: int, new_tokens: int, schedule: str | None = None,
                 prefill_width: int | None = None, torch_glue: bool = True):
    """Resident greedy decode on random-init weights: chunked prefill of a random
    prompt, then ``new_tokens`` graph replays with no host read in between."""
    from deepfold_amd import decodev2 as dv2

    spec = {"3b": dv2.QWEN25_3B, "14b": dv2.QWEN25_14B, "20b": dv2.INTERNLM25_20B,
            "32b": dv2.QWEN25_32B}[spec_name]
    t0 = time.perf_counter()
    weights = dv2.DeviceWeights.random(spec, seed=2026)
    torch.cuda.synchronize()
    load_s = time.perf_counter() - t0
    state = dv2.DecodeState.allocate(spec, device="cuda")
    g = torch.Generator(device="cpu")
    g.manual_seed(7)
    prompt = torch.randint(0, spec.vocab, (prompt_len,), generator=g).tolist()
    # prefill: the token-major torch glue of the reference's sequence (32-position chunks;
    # timed on request only, it is slow), then the feature-major launches (first pass
    # captures one graph per chunk width, the timed pass replays them)
    prefill_glue_ms = None
    if torch_glue:
        state.reset()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        dv2.consume_prompt(state, weights, prompt)
        torch.cuda.synchronize()
        prefill_glue_ms = (time.perf_counter() - t0) * 1e3
    pre = dv2.ChunkPrefill(state, weights, width=prefill_width)
    width = pre.width
    state.reset()
    dv2.consume_prompt(state, weights, prompt, prefill=pre)
    state.reset()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    dv2.consume_prompt(state, weights, prompt, prefill=pre)
    torch.cuda.synchronize()
    prefill_ms = (time.perf_counter() - t0) * 1e3
    del pre
    state.token.copy_(state.next_token)
    graph = dv2.capture_greedy(state, weights, warmup=2, schedule=schedule)
    torch.cuda.synchronize()
    start_pos = int(state.position.item())
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(new_tokens):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    dev_ms = e0.elapsed_time(e1)
    end_pos = int(state.position.item())
    assert end_pos == start_pos + new_tokens
    # the same replays with the host reading every token id before it launches the next
    # step (gpu/decodev2/profile_step.py:409-483 reports both)
    n_read = min(32, new_tokens)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(n_read):
        graph.replay()
        int(state.next_token.item())
    host_read_ms = (time.perf_counter() - t0) * 1e3 / n_read
    # eager step for comparison (a few tokens)
    t0 = time.perf_counter()
    for _ in range(8):
        dv2.greedy_decode(state, weights, schedule=schedule)
    torch.cuda.synchronize()
    eager_ms = (time.perf_counter() - t0) * 1e3 / 8
    ms_tok = dev_ms / new_tokens
    mean_ctx = (start_pos + end_pos) / 2.0
    bytes_tok = spec.weight_bytes_per_token() + spec.kv_bytes(mean_ctx)
    roof_ms = bytes_tok / (HBM_PEAK_GBPS * 1e9) * 1e3
    out = {
        "model": spec.name, "layers": spec.n_layers, "hidden": spec.hidden, "ffn": spec.intermediate,
        "vocab": spec.vocab, "max_seq": spec.max_seq, "prompt_tokens": prompt_len,
        "new_tokens": new_tokens, "context_start": start_pos, "context_end": end_pos,
        "tok_s": 1e3 / ms_tok, "ms_per_token": ms_tok, "tok_s_host_clock": new_tokens / wall,
        "tok_s_host_read": 1e3 / host_read_ms, "eager_ms_per_token": eager_ms, "prefill_ms": prefill_ms,
        "prefill_torch_glue_ms": prefill_glue_ms, "prefill_chunk_tokens": width,
        "prefill_tok_s": prompt_len / (prefill_ms * 1e-3),
        "weight_gb_per_token": spec.weight_bytes_per_token() / 1e9,
        "kv_mb_per_token_mean": spec.kv_bytes(mean_ctx) / 1e6,
        "roofline_ms_per_token": roof_ms, "roofline_tok_s": 1e3 / roof_ms,
        "roofline_frac": roof_ms / ms_tok, "achieved_gbps": bytes_tok / (ms_tok * 1e-3) / 1e9,
        "weights_load_s": load_s,
        "gemv_levels": "binary16 levels (default)",
    }
    del graph, state, weights
    torch.cuda.empty_cache()
    return out


def cpu_baseline(m: int, k: int, budget_s: float = 12.0) -> dict:
    """The reference's CPU path for this layer, restated by the oracle: decode the
    whole matrix to fp32, then an fp32 matmul.  Timed on all host threads the
    OpenMP runtime offers and on one thread."""
    import numpy as np

    from oracle import nf4_oracle as oc

    rng = np.random.default_rng(0)
    w = (rng.standard_normal((m, k)) * 0.02).astype(np.float32)
    packed, scale = oc.c_encode(w)
    x = oc.bf16_round(rng.standard_normal((k, 1)).astype(np.float32))
    L = oc.lib()
    scratch = np.empty((m, k), dtype=np.float32)
    y = np.empty((m, 1), dtype=np.float32)
    s16 = scale.view(np.uint16)

    def run_for(threads: int, budget: float):
        L.or_set_threads(threads)
        L.or_linear_two_pass(packed.ctypes.data, s16.ctypes.data, m, k, x.ctypes.data, 1,
                             scratch.ctypes.data, y.ctypes.data)
        n = 0
        t0 = time.perf_counter()
        while True:
            L.or_linear_two_pass(packed.ctypes.data, s16.ctypes.data, m, k, x.ctypes.data, 1,
                                 scratch.ctypes.data, y.ctypes.data)
            n += 1
            dt = time.perf_counter() - t0
            if dt >= budget:
                return dt / n, n

    def fused_for(threads: int, budget: float):
        """decode + dot in one pass over the packed bytes (no fp32 copy of W)"""
        L.or_set_threads(threads)
        xf = np.ascontiguousarray(x.reshape(-1))
        L.or_gemv_fused(packed.ctypes.data, s16.ctypes.data, m, k, xf.ctypes.data, y.ctypes.data)
        n = 0
        t0 = time.perf_counter()
        while True:
            L.or_gemv_fused(packed.ctypes.data, s16.ctypes.data, m, k, xf.ctypes.data, y.ctypes.data)
            n += 1
            dt = time.perf_counter() - t0
            if dt >= budget:
                return dt / n

    cores = min(int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or (os.cpu_count() or 1), 64)
    t_all, n_all = run_for(cores, budget_s * 0.5)
    t_one, n_one = run_for(1, budget_s * 0.35)
    t_fused = fused_for(cores, budget_s * 0.15)
    by = algorithmic_bytes(m, k)
    return {
        "value": by / t_all / 1e9,
        "unit": "GB/s",
        "cores": cores,
        "kind": "port",
        "sample": f"{n_all} passes of the two-pass CPU linear (decode to fp32, then fp32 matmul) "
                  f"over the same {m}x{k} layer",
        "us_per_gemv": t_all * 1e6,
        "single_thread_gbps": by / t_one / 1e9,
        "single_thread_us_per_gemv": t_one * 1e6,
        "fused_decode_dot_gbps": by / t_fused / 1e9,
        "fused_decode_dot_us_per_gemv": t_fused * 1e6,
    }


def bench_ring(torch, nf4, n_matrices: int = 192, distinct: int = 48, forwards: int = 3):
    """Streaming variant at model scale: the FFN matrices of the 32B architecture (64 layers
    x gate, up, down = 192 matrices of 27648x5120 codes, 75.2 MB each, 14.4 GB per token)
    live in pinned host memory and pass through two device slots, one GEMV each.  The tape
    has 192 entries over ``distinct`` different host images (the bytes that cross the bus per
    token are the same; holding 192 distinct images would only pin more host memory)."""
    from deepfold_amd import ring as rg

    m, k = 27648, 5120
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    images = []
    for i in range(distinct):
        w = torch.randn((m, k), generator=g, device="cuda", dtype=torch.float32) * 0.02
        packed, scale = nf4.nf4_quantize(w)
        del w
        images.append(rg.HostImage.from_blobs(packed, scale, k))
        del packed, scale
    tape = [rg.StreamedMatrix.on_host(f"ffn{i}", images[i % distinct]) for i in range(n_matrices)]
    ring = rg.CopyRing(rg.SlotPair(images[0].nbytes, "cuda"))
    x = torch.randn(k, generator=g, device="cuda").to(torch.bfloat16)

    def forward():
        ring.arm(tape)
        ring.prefetch()
        for mat in tape:
            rg.streamed_linear(ring, mat, x)
        ring.prefetch_next()

    forward()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(forwards):
        forward()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / forwards
    nbytes = n_matrices * images[0].nbytes
    return {
        "workload": f"{n_matrices} x NF4 [{m},{k}] (the 32B architecture's FFN matrices of one token, "
                    f"{distinct} distinct host images) streamed from pinned host memory through 2 "
                    "slots, one GEMV each",
        "slot_bytes": images[0].nbytes,
        "bytes_per_forward": nbytes,
        "ms_per_forward": dt * 1e3,
        "h2d_gbps": nbytes / dt / 1e9,
        "pinned": rg.is_pinned(images[0].arena),
        "copies_per_forward": n_matrices,
    }


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--copies", type=int, default=16, help="distinct weight copies to rotate through")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-decode", action="store_true", help="skip the model decode leg")
    ap.add_argument("--no-prefill", action="store_true", help="skip the prefill GEMM sweep")
    ap.add_argument("--no-ring", action="store_true", help="skip the host-streaming ring leg")
    ap.add_argument("--prefill-layers", default="", help="comma list of qkv,o,gate_up,down (default all)")
    ap.add_argument("--prefill-widths", default="8,16,32,64", help="chunk widths of the prefill sweep")
    ap.add_argument("--decode-models", default="3b,14b,20b,32b", help="comma list of 3b,14b,20b,32b")
    ap.add_argument("--no-shapes", action="store_true", help="skip the GEMV sweep over other shapes")
    ap.add_argument("--no-layer", action="store_true",
                    help="skip the five launches of a 14B decode layer measured one by one")
    ap.add_argument("--schedule", default=None, help="decode launch schedule: plain or fold_rms")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="MiB",
                    help="first run four plain device copies of this size (a kernel of known "
                         "traffic to scale hardware counters by)")
    ap.add_argument("--prompt", type=int, default=None,
                    help="prompt tokens of every decode model (default: each model's own "
                         "configuration, see DECODE_CONFIGS)")
    ap.add_argument("--new-tokens", type=int, default=None)
    ap.add_argument("--prefill-width", type=int, default=None,
                    help="tokens per prefill chunk of the feature-major prefill (default 64; the "
                         "reference's chunks are 32)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build drives one GPU; --gpus N with N > 1 is not supported "
              "(nothing on this path shards across devices).", file=sys.stderr)
        return 2

    import torch

    import deepfold_amd.nf4 as nf4

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    torch.cuda.set_device(0)

    if args.copy_calibration > 0:
        src = torch.empty(args.copy_calibration << 20, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    ms, eager_ms, copies, by, forms = bench_gemv(torch, nf4, args.steps, args.warmup, args.copies)
    achieved = by / (ms * 1e-3) / 1e9

    def roofline_of(ms_launch: float, kernel: str, multiplies: str) -> dict:
        a = by / (ms_launch * 1e-3) / 1e9
        return {"bound": "hbm", "achieved": a, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": a / HBM_PEAK_GBPS, "traffic": None, "kernel": kernel,
                "multiplies": multiplies, "us_per_launch": ms_launch * 1e3,
                "algorithmic_bytes_per_launch": by}

    out = {
        "metric": "nf4_gemv_hbm_gbps",
        "value": achieved,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        # what the timed kernel multiplies: NF4 levels rounded to binary16 times the bf16
        # activations held as binary16 (exactly: a power of two puts the largest in range),
        # exact products, fp32 accumulation; bf16 in, bf16 out
        "dtype": "f16",
        "dtype_note": "binary16 level pairs x bf16 activations staged as binary16 (v_dot2c_f32_f16), "
                      "fp32 accumulate, one bf16 rounding of y",
        "data": "synthetic",
        "config": {
            "workload": f"decode GEMV x[1,{K}] bf16 @ W[{M},{K}] NF4 group-64, {copies} rotating weight "
                        f"copies ({copies * by / 2**20:.0f} MiB)",
            "M": M, "K": K, "N": 1,
        },
        "eager_ms_per_step": eager_ms,
        "roofline": {
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS,
            "traffic": GEMV_TRAFFIC_BYTES if (M, K) == (13824, 5120) else None,
            "kernel": "gemv_ring_rows<5,3,true> (binary16 levels)",
            "algorithmic_bytes_per_launch": by,
            # the figures of the other legs that belong beside this one (each is also given in
            # full further down the line): fractions of 8 TB/s for the same launches through the
            # other two kernel forms, and of each model's bandwidth roofline for the decode legs
            "other": {
                "two_term_frac": by / (forms["two_term"] * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                "two_term_us_per_launch": forms["two_term"] * 1e3,
                "one_term_frac": by / (forms["one_term"] * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                "one_term_us_per_launch": forms["one_term"] * 1e3,
                "fp32_levels_frac": by / (forms["fp32_levels"] * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                "fp32_levels_us_per_launch": forms["fp32_levels"] * 1e3,
                "window_launches": args.steps * max(1, -(-MIN_WINDOW_LAUNCHES // args.steps)),
            },
        },
        # the same launches on the same copies through the other kernel forms
        "roofline_two_term": roofline_of(forms["two_term"], "gemv_ring_rows<5,2,true> (head + tail bf16 levels)",
                                         "two bf16 terms per level x bf16 activations"),
        "roofline_one_term": roofline_of(forms["one_term"], "gemv_ring_rows<5,1,true> (one bf16 level)",
                                         "bf16 levels x bf16 activations"),
        "roofline_fp32_levels": roofline_of(forms["fp32_levels"], "gemv_stream (plain)",
                                            "fp32 levels x fp32-widened activations, 128-bit loads"),
    }
    if not args.no_shapes:
        out["gemv_shapes"] = bench_gemv_shapes(torch, nf4)
        for row in out["gemv_shapes"]:
            out["roofline"]["other"][f"gemv_{row['M']}x{row['K']}_frac"] = row["hbm_frac"]
    if not args.no_layer:
        out["layer_launches"] = bench_layer_launches(torch, nf4)
        out["roofline"]["other"]["layer_14b_sum_us"] = sum(
            r["us"] for r in out["layer_launches"] if "2047" not in r["launch"])
    if not args.no_decode:
        rows = []
        for name in (n.strip() for n in args.decode_models.split(",")):
            if not name:
                continue
            prompt, width, new = DECODE_CONFIGS[name]
            prompt = args.prompt if args.prompt is not None else prompt
            new = args.new_tokens if args.new_tokens is not None else new
            width = args.prefill_width if args.prefill_width is not None else width
            rows.append(bench_decode(torch, name, prompt, new, args.schedule, width,
                                     torch_glue=(name == "14b")))
            if name == "14b":
                # the same model with the other two forms of the levels: two bf16 terms (more
                # exact, 8-byte lookups) and one bf16 term (less exact)
                for form, label in (("two_term", "two bf16 terms (CHR_NF4_GEMV_TERMS=2)"),
                                    ("one_term", "one bf16 term (CHR_NF4_GEMV_TERMS=1)")):
                    with gemv_form(form):
                        other = bench_decode(torch, name, prompt, new, args.schedule, width, torch_glue=False)
                    other["gemv_levels"] = label
                    rows.append(other)
        out["decode"] = rows
        for row in rows:
            key = row["model"].lower().replace(" ", "_").replace(".", "")
            if row["gemv_levels"].startswith("one"):
                key += "_one_term"
            elif row["gemv_levels"].startswith("two"):
                key += "_two_term"
            out["roofline"]["other"][f"decode_{key}_roofline_frac"] = row["roofline_frac"]
            out["roofline"]["other"][f"decode_{key}_tok_s"] = row["tok_s"]
    if not args.no_prefill:
        only = [v.strip() for v in args.prefill_layers.split(",") if v.strip()]
        widths = tuple(int(v) for v in args.prefill_widths.split(",") if v.strip())
        out["prefill"] = bench_prefill(torch, nf4, only, widths)
    if not args.no_ring:
        out["ring"] = bench_ring(torch, nf4)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(M, K)
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
