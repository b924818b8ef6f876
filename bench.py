#!/usr/bin/env python3
"""Decode-attention benchmark over the hybrid quantized KV cache (one MI355X).

A step is ONE decode-attention layer-step (q.K^T over every precision class, scale+softmax, p.V over
every class, split-K combine) on one layer's cache.  Steps cycle through ``--layers`` distinct layer
caches (default 32, like the 32 decoder layers of Llama-3.1-8B) so no step finds its cache in L2 or in
the 256 MB Infinity Cache.  Inputs are resident in HBM before the timed region.

Prints ONE JSON line: metric/value are microseconds per layer-step; ``roofline`` prices the dominant
kernel's algorithmic bytes against the 8 TB/s HBM peak using its average duration measured live with
HIP events; ``cpu_baseline`` times the CPU restatement of the reference's unpack + dequant +
torch.matmul path on the same layer-0 inputs on the host cores.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
METRIC = "us/layer decode-attn & achieved HBM GB/s (% of peak) at 32k ctx, 1 GPU"

WORKLOADS = {
    "c1": "Llama-3.1-8B shape, B=1, ctx 4096: 3968 tokens 2-bit + 128 fp16 residual",
    "c2": "Llama-3.1-8B shape, B=1, ctx 32768 hybrid: fp16 5% / 8-bit 15% / 4-bit 30% / 2-bit 30% / evicted 20%",
    "c4": "Qwen3-8B shape, B=8, ctx 65536 hybrid: fp16 10% / 4-bit 20% / 2-bit 50% / evicted 20%",
    "c5": "decode-attention share of config 5: Llama-3.1-8B shape, B=4, ctx 131072 hybrid: fp16 2% / 8-bit 3% / 4-bit 25% / 2-bit 50% / evicted 20% (2.56 bit average), 32 layers resident",
    "c3": "quantize-and-pack: 8 KV heads x 128 x 8192 new fp16 tokens appended at token 24576 of a 32768-token cache",
    "prompt": "prompt side: causal attention over a 32768-token prompt (B=1, Hq=32, Hkv=8, D=128, fp16) + the last 20 rows' probabilities",
}


def kernel_source_sha16() -> str:
    """Hash of the HIP sources the decode-attention kernels are built from (attn.hip and the headers): recorded next
    to counter-derived figures so that a figure measured on other kernels is recognised as stale."""
    import hashlib
    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "hqekv_amd", "csrc")
    for name in sorted(os.listdir(csrc)):
        if name == "attn.hip" or name.endswith(".h"):
            h.update(name.encode())
            h.update(open(os.path.join(csrc, name), "rb").read())
    return h.hexdigest()[:16]


def cpu_model() -> str:
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def recorded_traffic(workload: str, kernel: str):
    """HBM bytes per launch of ``kernel`` from the committed rocprofv3 --pmc summary, or (None, why) when that
    summary was taken on other kernel sources than the ones this run uses.  The counters need the profiler, so
    the figure is a recorded one, never measured by the run that prints it."""
    path = os.path.join(ROOT, "profiles", "pmc_traffic.json")
    try:
        rec = json.load(open(path))
    except (OSError, ValueError):
        return None, "profiles/pmc_traffic.json missing"
    now = kernel_source_sha16()
    if rec.get("kernel_source_sha16") != now:
        return None, f"profiles/pmc_traffic.json was recorded on kernel sources {rec.get('kernel_source_sha16')}, this run uses {now}"
    val = rec.get(workload, {}).get(kernel)
    return val, f"recorded: profiles/pmc_traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on kernel sources {now})"


def side_bytes(pkv, k_side: bool) -> int:
    """Algorithmic bytes of the K side (q.K^T launch) or V side (p.V launch) of one layer-step."""
    if k_side:
        slots = (0, 1, 4, 5, 6, 7, 12, 13, 14, 15, 20, 21, 22, 23, 28, 29, 30, 31, 39)
    else:
        slots = (2, 3, 8, 9, 10, 11, 16, 17, 18, 19, 24, 25, 26, 27, 32, 33, 34, 35, 40)
    return sum(pkv[i].numel() * pkv[i].element_size() for i in slots if torch.is_tensor(pkv[i]))


def build_layers(name: str, n_layers: int, dev):
    from hqekv_amd import synth
    from hqekv_amd.pack_unpack import uniform_group_quantize_pack_last_dim as hip_quant
    cfg = synth.CONFIGS[name]
    layers = []
    q0 = cpu_cache = None
    for l in range(n_layers):
        if l == 0:
            # layer 0 is the CPU-seeded configuration, also handed to the CPU baseline
            q, K, V = synth.make_qkv(cfg["B"], cfg["Hq"], cfg["Hkv"], cfg["T"], cfg["D"], cfg["seed"])
            q, K, V = q.to(dev), K.to(dev), V.to(dev)
        else:
            g = torch.Generator(device=dev).manual_seed(cfg["seed"] + 1000 * l)
            K = torch.randn(cfg["B"], cfg["Hkv"], cfg["T"], cfg["D"], generator=g, device=dev)
            V = torch.randn(cfg["B"], cfg["Hkv"], cfg["T"], cfg["D"], generator=g, device=dev).half()
            for c in synth.OUTLIER_CHANNELS:
                K[..., c] *= 10.0
            K = K.half()
            q = torch.randn(cfg["B"], cfg["Hq"], 1, cfg["D"], generator=g, device=dev).half()
        classes = synth.split_blocks(cfg["T"] - cfg["residual"], cfg["fractions"], cfg["seed"] + 1000 * l)
        cache = synth.build_cache(K, V, classes, cfg["residual"], hip_quant)
        layers.append((q, cache))
        del K, V
    return layers


def time_region(fn, sync):
    sync()
    t0 = time.perf_counter()
    fn()
    sync()
    return time.perf_counter() - t0


def event_avg_us(launch, n_launches: int, reps: int) -> float:
    """Average duration of one launch: HIP events on the launch stream around back-to-back launches."""
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = []
    for _ in range(reps):
        e0.record()
        launch()
        e1.record()
        e1.synchronize()
        best.append(e0.elapsed_time(e1) * 1e3 / n_launches)
    return statistics.median(best)


def cpu_baseline(name: str, n_iter: int = 5, gpu_layer0=None):
    """The reference's CPU-expressible path (unpack + dequant + torch.matmul) on layer 0.  With several batch
    rows the sample is batch row 0 of the GPU's own layer-0 cache (copied to the host), so the result also
    checks the GPU output of that row at full size."""
    from hqekv_amd import synth
    from oracle import hqe_oracle as O
    cores = min(16, os.cpu_count() or 1)
    torch.set_num_threads(cores)
    cfg = synth.CONFIGS[name]
    B = cfg["B"]
    sample = "one layer-step, all batch rows"
    scale = 1.0
    if B > 1 and gpu_layer0 is not None:  # bounded sample: one batch row, scaled by B
        sample = f"one layer-step of ONE batch row (row 0 of the GPU's layer-0 cache), time x{B}"
        scale = float(B)
        q_dev, pkv_dev = gpu_layer0
        q = q_dev[:1].cpu()
        cache = tuple((x[:1].cpu() if x.dim() == 4 else x.cpu()) if torch.is_tensor(x) else x for x in pkv_dev)
    else:
        q, K, V = synth.make_qkv(cfg["B"], cfg["Hq"], cfg["Hkv"], cfg["T"], cfg["D"], cfg["seed"])
        classes = synth.split_blocks(cfg["T"] - cfg["residual"], cfg["fractions"], cfg["seed"])
        cache = synth.build_cache(K, V, classes, cfg["residual"], O.uniform_group_quantize_pack_last_dim)
    times = []
    ref = None
    for i in range(n_iter + 1):
        t0 = time.perf_counter()
        ref = O.qkv_matmul(q, cache, None, cfg["D"], use_mask=False)
        if i:
            times.append(time.perf_counter() - t0)
    return dict(value=statistics.median(times) * 1e6 * scale, unit="us/layer", cores=cores, cpu_model=cpu_model(),
                kind="port", sample=f"{sample}; median of {n_iter} after 1 warm-up; torch {torch.__version__} CPU ops"), (q, cache, ref)


def bench_quantize(args):
    """Config 3: K (per channel, read in place from token-major memory) and V (per token) of 8192 new
    tokens quantised at 2/4/8 bit straight into windows of capacity-sized cache buffers."""
    from hqekv_amd import synth
    from hqekv_amd.pack_unpack import quantize_pack_into
    dev = torch.device("cuda:0")
    B, H, D, Tn, off, cap = 1, 8, 128, 8192, 24576, 32768
    n_copies = 8  # distinct inputs so no step finds its input in cache
    ins = []
    for c in range(n_copies):
        _, K, V = synth.make_qkv(B, 32, H, Tn, D, 1237 + 1000 * c) if c == 0 else (None, None, None)
        if c:
            g = torch.Generator(device=dev).manual_seed(1237 + 1000 * c)
            K = torch.randn(B, H, Tn, D, generator=g, device=dev)
            for ch in synth.OUTLIER_CHANNELS:
                K[..., ch] *= 10.0
            K = K.half()
            V = torch.randn(B, H, Tn, D, generator=g, device=dev).half()
        ins.append((K.to(dev), V.to(dev)))
    bufs = {}
    for bit in (2, 4, 8):
        pf = 32 // bit
        bufs[bit] = dict(
            kc=torch.zeros(B, H, D, cap // pf, dtype=torch.int32, device=dev),
            ks=torch.zeros(B, H, D, cap // 32, dtype=torch.float16, device=dev),
            kz=torch.zeros(B, H, D, cap // 32, dtype=torch.float16, device=dev),
            vc=torch.zeros(B, H, cap, D // pf, dtype=torch.int32, device=dev),
            vs=torch.zeros(B, H, cap, D // 32, dtype=torch.float16, device=dev),
            vz=torch.zeros(B, H, cap, D // 32, dtype=torch.float16, device=dev))

    def step(i, bit):
        K, V = ins[i % n_copies]
        b = bufs[bit]
        pf = 32 // bit
        quantize_pack_into(K.transpose(2, 3), bit, b["kc"][..., off // pf:], b["ks"][..., off // 32:], b["kz"][..., off // 32:])
        quantize_pack_into(V, bit, b["vc"][:, :, off:], b["vs"][:, :, off:], b["vz"][:, :, off:])

    def k_call(i, bit):
        b = bufs[bit]
        quantize_pack_into(ins[i][0].transpose(2, 3), bit, b["kc"][..., off // (32 // bit):], b["ks"][..., off // 32:], b["kz"][..., off // 32:])

    def v_call(i, bit):
        b = bufs[bit]
        quantize_pack_into(ins[i][1], bit, b["vc"][:, :, off:], b["vs"][:, :, off:], b["vz"][:, :, off:])

    def graph_of(fn):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            fn()
        g.replay()
        torch.cuda.synchronize()
        return g

    res = {}
    for bit in (2, 4, 8):
        for i in range(args.warmup):
            step(i, bit)
        torch.cuda.synchronize()
        # launches replayed from a HIP graph, so the figures are the kernels' and not the host's
        g_both = graph_of(lambda: [step(i, bit) for i in range(n_copies)])
        g_k = graph_of(lambda: [k_call(i, bit) for i in range(n_copies)])
        g_v = graph_of(lambda: [v_call(i, bit) for i in range(n_copies)])
        reps = max(1, args.steps // n_copies)
        t0 = time.perf_counter()
        for _ in range(reps):
            g_both.replay()
        torch.cuda.synchronize()
        us = (time.perf_counter() - t0) / (reps * n_copies) * 1e6
        k_us = event_avg_us(g_k.replay, n_copies, 9)
        v_us = event_avg_us(g_v.replay, n_copies, 9)
        elems = B * H * D * Tn
        nbytes = elems * 2 + elems * bit // 8 + elems // 32 * 4     # per tensor: read fp16, write codes + scale + zero
        res[bit] = dict(us_k_plus_v=round(us, 2), k_us=round(k_us, 2), v_us=round(v_us, 2), bytes_per_tensor=nbytes,
                        k_GBps=round(nbytes / k_us / 1e3, 1), v_GBps=round(nbytes / v_us / 1e3, 1))
    # bit-exactness of what was appended (2-bit, first input) against the oracle on the CPU
    from oracle import hqe_oracle as O
    step(0, 2)
    torch.cuda.synchronize()
    K0, V0 = ins[0][0].cpu(), ins[0][1].cpu()
    okc, oks, okz = O.uniform_group_quantize_pack_last_dim(K0.transpose(2, 3).contiguous(), 32, 2)
    ovc, ovs, ovz = O.uniform_group_quantize_pack_last_dim(V0, 32, 2)
    b = bufs[2]
    exact = bool(torch.equal(b["kc"][..., off // 16:].cpu(), okc) and torch.equal(b["ks"][..., off // 32:].cpu(), oks)
                 and torch.equal(b["kz"][..., off // 32:].cpu(), okz) and torch.equal(b["vc"][:, :, off:].cpu(), ovc)
                 and torch.equal(b["vs"][:, :, off:].cpu(), ovs) and torch.equal(b["vz"][:, :, off:].cpu(), ovz))
    # CPU baseline: the oracle's quantiser (torch CPU ops) on a bounded sample, one KV head of K and of V
    cpu = None
    if not args.no_cpu:
        cores = min(16, os.cpu_count() or 1)
        torch.set_num_threads(cores)
        ks, vs = K0[:, :1].transpose(2, 3).contiguous(), V0[:, :1].contiguous()
        times = []
        for i in range(4):
            t0 = time.perf_counter()
            O.uniform_group_quantize_pack_last_dim(ks, 32, 2)
            O.uniform_group_quantize_pack_last_dim(vs, 32, 2)
            if i:
                times.append(time.perf_counter() - t0)
        cpu = dict(value=statistics.median(times) * 1e6 * H, unit="us", cores=cores, cpu_model=cpu_model(), kind="port",
                   sample=f"K + V of ONE of the {H} KV heads at 2 bit, time x{H}; median of 3 after 1 warm-up")
    dom = max(res[2]["k_us"], res[2]["v_us"])
    out = {"metric": "us per quantize-and-pack of 8192 new tokens (K + V, 2-bit) & GB/s", "value": res[2]["us_k_plus_v"],
           "unit": "us", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": round(res[2]["us_k_plus_v"] / 1e3, 6), "higher_is_better": False, "scaling": "weak",
           "vs_baseline": None, "dtype": "f16", "data": "synthetic",
           "config": {"workload": f"c3: {WORKLOADS['c3']}", "launch": "hip-graph replay"},
           "per_bit": res, "bit_exact_vs_oracle_2bit": exact,
           "roofline": {"bound": "hbm", "kernel": "quant_k_tokenmajor_kernel<2>" if res[2]["k_us"] >= res[2]["v_us"] else "quant_rows_kernel<2>",
                        "achieved": round(res[2]["bytes_per_tensor"] / dom / 1e3, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                        "frac": round(res[2]["bytes_per_tensor"] / dom / 1e3 / HBM_PEAK_GBPS, 4), "traffic": None}}
    if cpu is not None:
        out["cpu_baseline"] = cpu
    print(json.dumps(out))



# ------------------------------------------------------------------------------------------------ prompt side
def measure_prompt(T: int, steps: int, warm: int) -> dict:
    """Causal prompt attention (B=1, Hq=32, Hkv=8, D=128, fp16) and the last 20 rows' probabilities on the library's
    matrix-core kernels, torch's fused attention on the same tensors beside it."""
    import math
    from hqekv_amd.prompt_attention import prompt_attention, prompt_last_rows
    dev = torch.device("cuda:0")
    B, Hq, Hkv, D, R = 1, 32, 8, 128, 20
    g = torch.Generator(device=dev).manual_seed(1241)
    q = torch.randn(B, Hq, T, D, generator=g, device=dev, dtype=torch.float16)
    k = torch.randn(B, Hkv, T, D, generator=g, device=dev, dtype=torch.float16)
    v = torch.randn(B, Hkv, T, D, generator=g, device=dev, dtype=torch.float16)
    scale = 1.0 / math.sqrt(D)

    def timed(fn):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(steps):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / steps

    def fused(): return torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, scale=scale, enable_gqa=True)
    ms = timed(lambda: prompt_attention(q, k, v, scale))
    ms_rows = timed(lambda: prompt_last_rows(q, k, scale, R))
    ms_torch = timed(fused)
    flop = 4.0 * B * Hq * (T * (T + 1) / 2) * D   # two products, causal: T (T + 1) / 2 (query, key) pairs
    diff = float((prompt_attention(q, k, v, scale).float() - fused().float()).abs().max())
    torch.cuda.synchronize()
    tf = flop / (ms * 1e-3) / 1e12
    return {"T": T, "steps": steps, "warmup": warm, "ms": round(ms, 4), "TFLOP/s": round(tf, 1), "last_rows_ms": round(ms_rows, 4),
            "torch_fused_attention": {"ms": round(ms_torch, 4), "TFLOP/s": round(flop / (ms_torch * 1e-3) / 1e12, 1),
                                      "note": "torch.nn.functional.scaled_dot_product_attention(is_causal, enable_gqa) on the same tensors, same process"},
            "max_abs_difference_from_torch": diff,
            "roofline": {"bound": "mfma", "kernel": "prompt_attn_kernel<true>", "achieved": round(tf, 1), "peak": 2500.0, "unit": "TFLOP/s",
                         "frac": round(tf / 2500.0, 4), "traffic": None}}


def bench_prompt(args):
    T = args.prompt_len if args.prompt_len != 131072 else 32768
    steps, warm = max(1, min(args.steps, 20)), max(1, min(args.warmup, 3))
    m = measure_prompt(T, steps, warm)
    print(json.dumps({
        "metric": "TFLOP/s of the causal prompt attention (fp16, fp32 accumulation)", "value": m["TFLOP/s"], "unit": "TFLOP/s",
        "n_gpus": 1, "steps": steps, "warmup": warm, "ms_per_step": m["ms"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"prompt: {WORKLOADS['prompt']}", "T": T},
        "last_rows_ms": m["last_rows_ms"], "torch_fused_attention": m["torch_fused_attention"],
        "max_abs_difference_from_torch": m["max_abs_difference_from_torch"], "roofline": m["roofline"],
    }))


# ------------------------------------------------------------------------------------------------ config 5
# End-to-end greedy decode of a random-init Llama-3.1-8B (bf16 weights) on the HqeKV cache.  The model around
# the attention path (embedding, RMSNorm, projections, rotary embedding, MLP, lm_head) is plain torch: it is
# the load the path runs under, not part of it.

class _RandomLlama:
    HID, FFN, VOCAB, HQ, HKV, D, THETA, EPS = 4096, 14336, 128256, 32, 8, 128, 500000.0, 1e-5

    def __init__(self, n_layers: int, dev, seed: int = 0):
        g = torch.Generator(device=dev).manual_seed(seed)

        def w(*shape):
            return torch.empty(*shape, dtype=torch.bfloat16, device=dev).normal_(0.0, 0.02, generator=g)

        self.dev, self.n_layers = dev, n_layers
        self.embed, self.lm_head = w(self.VOCAB, self.HID), w(self.VOCAB, self.HID)
        self.norm_f = torch.ones(self.HID, dtype=torch.bfloat16, device=dev)
        self.layers = []
        for _ in range(n_layers):
            self.layers.append(dict(
                n1=torch.ones(self.HID, dtype=torch.bfloat16, device=dev),
                n2=torch.ones(self.HID, dtype=torch.bfloat16, device=dev),
                qkv=w((self.HQ + 2 * self.HKV) * self.D, self.HID), o=w(self.HID, self.HQ * self.D),
                gate_up=w(2 * self.FFN, self.HID), down=w(self.HID, self.FFN)))
        self.inv_freq = 1.0 / (self.THETA ** (torch.arange(0, self.D, 2, device=dev, dtype=torch.float32) / self.D))

    def rot(self, pos):
        """(cos, sin) tables (1, T, 1, D) for positions pos (T,), HF 'rotate_half' convention."""
        ang = pos.to(torch.float32)[:, None] * self.inv_freq[None, :]
        cos, sin = ang.cos(), ang.sin()
        return (torch.cat((cos, cos), -1)[None, :, None, :].to(torch.bfloat16),
                torch.cat((sin, sin), -1)[None, :, None, :].to(torch.bfloat16))

    def qkv(self, lw, x, rot):
        """x (B, T, HID) -> q (B,Hq,T,D), k, v (B,Hkv,T,D) fp16, rotary applied to q and k in one go."""
        F = torch.nn.functional
        B, T, _ = x.shape
        y = F.linear(F.rms_norm(x, (self.HID,), lw["n1"], self.EPS), lw["qkv"]).view(B, T, self.HQ + 2 * self.HKV, self.D)
        qk, h = y[:, :, : self.HQ + self.HKV], self.D // 2
        qk = (qk * rot[0] + torch.cat((-qk[..., h:], qk[..., :h]), -1) * rot[1]).transpose(1, 2).half()
        return qk[:, : self.HQ], qk[:, self.HQ:], y[:, :, self.HQ + self.HKV:].transpose(1, 2).half()

    def after_attention(self, lw, x, attn):
        """x (B,T,HID) residual stream, attn (B,Hq,T,D) fp16 -> new residual stream."""
        F = torch.nn.functional
        B, T, _ = x.shape
        x = x + F.linear(attn.transpose(1, 2).reshape(B, T, self.HQ * self.D).to(torch.bfloat16), lw["o"])
        gu = F.linear(F.rms_norm(x, (self.HID,), lw["n2"], self.EPS), lw["gate_up"])
        return x + F.linear(F.silu(gu[..., : self.FFN]) * gu[..., self.FFN:], lw["down"])

    def logits(self, x):
        F = torch.nn.functional
        return F.linear(F.rms_norm(x, (self.HID,), self.norm_f, self.EPS), self.lm_head)


def bench_end_to_end(args):
    from hqekv_amd.decode_layer import HqeAttentionLayer
    dev = torch.device("cuda:0")
    B, T0, NEW, NL = args.e2e_batch, args.prompt_len, args.new_tokens, args.layers or 32
    CH = 16384  # tokens per chunk of the prompt pass outside attention (bounds the MLP's intermediate)
    m = _RandomLlama(NL, dev)
    # shares of all tokens: evicted 20 %, 4-bit 48 %, 2-bit 32 % (+ 64 fp16 tokens): 2.56 bit on average
    att = [HqeAttentionLayer(m.D, bit_0=0.20, bit_4=0.48, bit_2=0.32, bit_1=0.0) for _ in range(NL)]
    for a in att:
        a.set_max_length(T0 + NEW)
    g = torch.Generator(device=dev).manual_seed(1239)
    tokens = torch.randint(0, m.VOCAB, (B, T0), generator=g, device=dev)
    sync = torch.cuda.synchronize

    # ---- prompt pass, layer by layer over the whole prompt; each layer's cache is compressed right away
    t0 = time.perf_counter()
    x = m.embed[tokens]
    pos = torch.arange(T0, device=dev)
    caches, aux = [], None
    for l, lw in enumerate(m.layers):
        q = torch.empty(B, m.HQ, T0, m.D, dtype=torch.float16, device=dev)
        k = torch.empty(B, m.HKV, T0, m.D, dtype=torch.float16, device=dev)
        v = torch.empty(B, m.HKV, T0, m.D, dtype=torch.float16, device=dev)
        for c0 in range(0, T0, CH):
            qc, kc, vc = m.qkv(lw, x[:, c0:c0 + CH], m.rot(pos[c0:c0 + CH]))
            q[:, :, c0:c0 + CH], k[:, :, c0:c0 + CH], v[:, :, c0:c0 + CH] = qc, kc, vc
        del qc, kc, vc
        out, _, pkv, aux = att[l](q, k, v, None, None, aux if l > 0 else None)
        del q, k, v
        for c0 in range(0, T0, CH):
            x[:, c0:c0 + CH] = m.after_attention(lw, x[:, c0:c0 + CH], out[:, :, c0:c0 + CH])
        del out
        caches.append(pkv)
        sync()
        print(f"[c5] prompt pass layer {l + 1}/{NL} done, {time.perf_counter() - t0:.1f} s", file=sys.stderr, flush=True)
    nxt = m.logits(x[:, -1:]).argmax(-1)  # (B, 1)
    del x
    sync()
    prompt_s = time.perf_counter() - t0
    from hqekv_amd.attention import value_length
    kept = value_length(caches[0])

    # ---- greedy decode
    ev = [[(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(NL)]
          for _ in range(NEW)]
    step_ev = [torch.cuda.Event(enable_timing=True) for _ in range(NEW + 1)]
    sync()
    t0 = time.perf_counter()
    step_ev[0].record()
    for s in range(NEW):
        x = m.embed[nxt]
        rot = m.rot(torch.full((1,), T0 + s, device=dev))
        aux = None
        for l, lw in enumerate(m.layers):
            q, k, v = m.qkv(lw, x, rot)
            ev[s][l][0].record()
            out, _, caches[l], aux = att[l](q, k, v, None, caches[l], aux if l > 0 else None)
            ev[s][l][1].record()
            x = m.after_attention(lw, x, out)
        nxt = m.logits(x).argmax(-1)
        step_ev[s + 1].record()
    sync()
    decode_s = time.perf_counter() - t0
    attn_ms = [sum(a.elapsed_time(b) for a, b in row) for row in ev]
    step_ms = [step_ev[i].elapsed_time(step_ev[i + 1]) for i in range(NEW)]
    plain = [i for i in range(NEW) if (T0 + i + 1) % 32 != 0] or list(range(NEW))  # steps without a compression
    out = {
        "metric": "tokens/s, end-to-end greedy decode on the HqeKV cache (config 5)",
        "value": round(B * NEW / decode_s, 2), "unit": "tokens/s", "n_gpus": 1, "steps": NEW, "warmup": 0,
        "ms_per_step": round(decode_s / NEW * 1e3, 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16 cache / bf16 weights", "data": "synthetic",
        "config": {"workload": f"c5 end to end: random-init Llama-3.1-8B shape, {NL} layers, B={B}, prompt {T0} "
                               f"uniform-random token ids, {NEW} greedy tokens", "kept_tokens_after_prompt": kept,
                   "shares": "evicted 20 % / 4-bit 48 % / 2-bit 32 % / 64 tokens fp16 (2.56 bit average)"},
        "prompt_pass_s": round(prompt_s, 2),
        "attention_share_of_step_time": round(sum(attn_ms) / sum(step_ms), 4),
        "attention_ms_per_token_step": round(sum(attn_ms) / NEW, 3),
        "plain_steps": {"ms_per_token_step": round(sum(step_ms[i] for i in plain) / len(plain), 3),
                        "attention_ms": round(sum(attn_ms[i] for i in plain) / len(plain), 3)},
        "note": "attention = the whole cache-side layer call (hybrid q.K^T / p.V launches, ring update and, every "
                "32 tokens, the compression), measured with HIP events on the stream; the rest is torch",
    }
    print(json.dumps(out))


def measure_decode(workload: str, n_layers: int, K: int, W: int, args, dev):
    """Build ``n_layers`` distinct layer caches of ``workload`` and time the decode-attention layer-step on them.

    W untimed warm-up steps, then timed regions of EXACTLY K steps each (a barrier-free single process: synchronise on
    both sides), five of them; the figure is the median region.  Step i works on layer cache i mod n_layers, and the
    first timed step follows the last warm-up step's layer, so a timed step never finds its cache warm from the
    warm-up; between two regions a 512 MiB buffer is rewritten (untimed), which also empties the 256 MB memory-side
    cache.  Launches are replayed from HIP graphs (one of a whole cycle over the layers, one of the K mod n_layers
    steps that remain) unless --no-graph."""
    from hqekv_amd import _lib, synth
    from hqekv_amd.attention import DecodePlan, default_flags
    layers = build_layers(workload, n_layers, dev)
    plan_flags = default_flags() | _lib.qk_tiling(_lib.QK_TILINGS.get(args.qk_tiling, 0))
    plan_flags |= {"auto": 0, "mfma": _lib.DOT_MFMA, "valu": _lib.DOT_VALU}[args.dot]
    plan_flags |= {"auto": 0, "fold": _lib.FOLD_COMBINE, "separate": _lib.SEPARATE_COMBINE}[args.combine]
    plans = [DecodePlan(q, cache, flags=plan_flags) for q, cache in layers]
    qs = [q.contiguous() for q, _ in layers]
    cfg = synth.CONFIGS[workload]
    pkv0 = layers[0][1]
    alg_bytes = synth.algorithmic_bytes(pkv0, cfg["Hq"])
    k_bytes, v_bytes = side_bytes(pkv0, True), side_bytes(pkv0, False)
    sync = torch.cuda.synchronize

    def step(i):
        plans[i % n_layers].run(qs[i % n_layers])

    for i in range(W):
        step(i)
    sync()
    first = W % n_layers                    # the timed steps start where the warm-up stopped
    rounds, rem = divmod(K, n_layers)

    def graph_of(lo, n):
        if n == 0:
            return None
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for i in range(lo, lo + n):
                step(i)
        return g

    use_graph = not args.no_graph
    g_cycle = graph_of(first, n_layers) if use_graph and rounds else None
    g_rest = graph_of(first, rem) if use_graph and rem else None
    if use_graph:
        for g in (g_cycle, g_rest):
            if g is not None:
                g.replay()
        sync()

    def timed():
        if use_graph:
            for _ in range(rounds):
                g_cycle.replay()
            if g_rest is not None:
                g_rest.replay()
        else:
            for i in range(first, first + K):
                step(i)

    flush = torch.empty(512 << 20, dtype=torch.uint8, device=dev)
    regions, regions_host = [], []
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(5):
        # the rewrite of the flush buffer is queued right ahead of the timed steps, so they start on a busy GPU with
        # cold caches -- what a decode loop sees between two layers -- and not on one that has gone idle in a wait
        sync()
        flush.fill_(1)
        e0.record()
        timed()
        e1.record()
        sync()
        regions.append(e0.elapsed_time(e1) * 1e3 / K)
    for _ in range(5):   # the same K steps on the host's clock, synchronised on both sides
        regions_host.append(time_region(timed, sync) / K * 1e6)
    del flush
    # the figure is the GPU's time for the K steps (HIP events on the launch stream around exactly those steps);
    # the host's clock around a synchronised region adds the launch and wake-up latency of one graph replay, which
    # K = 20 steps do not amortise
    us_per_step = statistics.median(regions)
    us_per_step_host = statistics.median(regions_host)

    # per-kernel averages (HIP events on the launch stream), one kind of kernel back-to-back over all layers;
    # replayed from a HIP graph (unless --no-graph) so that the host's launch rate does not show in the
    # figure of a short kernel
    reps = 5
    fused = bool(plans[0].flags & _lib.FUSE_SOFTMAX)

    def part_us(launch_all, n=n_layers):
        if args.no_graph:
            return event_avg_us(launch_all, n, reps)
        launch_all()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            launch_all()
        return event_avg_us(g.replay, n, reps)

    qk_us = part_us(lambda: [p.run(q, only=_lib.ONLY_QK) for p, q in zip(plans, qs)])
    sm_us = 0.0
    if not fused:  # the general path has a softmax launch of its own; time it and take it out of the q.K^T figure
        sm_us = part_us(lambda: [p.run_softmax() for p in plans])
        qk_us -= sm_us
    pv_us = part_us(lambda: [p.run(q, only=_lib.ONLY_PV) for p, q in zip(plans, qs)])
    cb_us = part_us(lambda: [p.run(q, only=_lib.ONLY_COMBINE) for p, q in zip(plans, qs)])
    for p, q in zip(plans, qs):  # leave consistent outputs behind
        p.run(q)
    dominant = "qk_hybrid_kernel" if qk_us >= pv_us else "pv_hybrid_kernel"
    dom_us, dom_bytes = (qk_us, k_bytes) if qk_us >= pv_us else (pv_us, v_bytes)
    achieved = dom_bytes / (dom_us * 1e-6) / 1e9

    # the yardstick: a launch that only reads as many bytes as the dominant kernel must, from buffers as distinct as
    # the layer caches (1024 workgroups of 256 threads, 16-byte loads, eight in flight per lane), timed the same way
    lib = _lib.load()
    nb = (dom_bytes + 15) // 16 * 16
    bufs = [torch.empty(nb, dtype=torch.uint8, device=dev).fill_(i + 1) for i in range(n_layers)]
    sums = torch.zeros(1024, dtype=torch.int32, device=dev)

    def read_all():
        st = _lib.stream_ptr(dev)   # torch's current stream: the capture stream while a graph is recorded
        for b in bufs:
            _lib.check(lib.hqekv_selftest_stream_read(b.data_ptr(), nb, sums.data_ptr(), 1024, st), "stream_read")

    floor_us = part_us(read_all)
    del bufs
    traffic, traffic_source = recorded_traffic(workload, dominant)
    return dict(
        us_per_step=us_per_step, us_per_step_host=us_per_step_host, regions=[round(r, 3) for r in regions],
        alg_bytes=alg_bytes, cfg=cfg, layers=layers,
        plans=plans, qs=qs,
        config={"workload": f"{workload}: {WORKLOADS[workload]}", "B": cfg["B"], "Hq": cfg["Hq"],
                "Hkv": cfg["Hkv"], "head_dim": cfg["D"], "context": cfg["T"], "kept_tokens": pkv0[41],
                "layers_cycled": n_layers, "launch": "hip-graph replay" if use_graph else "eager",
                "timing": "median of 5 regions of `steps` steps, HIP events around the steps; 512 MiB rewritten "
                          "on the stream right before each region",
                "qk_tiling": args.qk_tiling, "dot": args.dot, "combine": args.combine,
                "softmax": "fused into the two GEMV launches" if fused else "separate launch",
                "algorithmic_bytes_per_step": alg_bytes},
        kernels_us={"qk_hybrid_kernel": round(qk_us, 3), "scale_softmax_kernel": round(sm_us, 3),
                    "pv_hybrid_kernel": round(pv_us, 3), "pv_combine_kernel": round(cb_us, 3)},
        roofline={"bound": "hbm", "kernel": dominant, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                  "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic,
                  "traffic_source": traffic_source, "bytes_per_launch": dom_bytes, "avg_us": round(dom_us, 3),
                  "launch_floor_us": round(floor_us, 3),
                  "launch_floor": "a launch that only reads bytes_per_launch bytes (hqekv_selftest_stream_read), same timing"})


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=640)
    ap.add_argument("--warmup", type=int, default=64)
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS))
    ap.add_argument("--layers", type=int, default=None, help="distinct layer caches cycled through")
    ap.add_argument("--qk-tiling", default="auto", choices=["auto", "8waves", "4waves", "wave512", "wave256"],
                    help="force one q.K^T tiling instead of the choice by launch size")
    ap.add_argument("--dot", default="auto", choices=["auto", "mfma", "valu"],
                    help="form of the inner products: matrix cores, vector ALU, or the library's default")
    ap.add_argument("--combine", default="auto", choices=["auto", "fold", "separate"],
                    help="who sums the split-K partials: the last p.V workgroup of each (b, kv head) or a launch of its own (auto: by launch size)")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true",
                    help="workload c2 only: skip the short configuration-4 measurement printed under 'extra'")
    ap.add_argument("--end-to-end", action="store_true",
                    help="workload c5 only: prompt pass + greedy decode of a random-init Llama-3.1-8B (takes minutes)")
    ap.add_argument("--prompt-len", type=int, default=131072)
    ap.add_argument("--new-tokens", type=int, default=256)
    ap.add_argument("--e2e-batch", type=int, default=4)
    ap.add_argument("--calibrate", action="store_true",
                    help="also run one plain 256 MiB device copy, the yardstick for rocprofv3 FETCH_SIZE / WRITE_SIZE")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs the decode-attention path on ONE GPU; --gpus {args.gpus} is not "
              "supported (no collectives or sharding are part of this path)", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(3)

    if args.workload == "c3":
        bench_quantize(args)
        return
    if args.workload == "prompt":
        bench_prompt(args)
        return
    if args.end_to_end:
        if args.workload != "c5":
            print("bench.py: --end-to-end belongs to --workload c5", file=sys.stderr)
            sys.exit(2)
        bench_end_to_end(args)
        return

    from hqekv_amd import synth
    from hqekv_amd.attention import DecodePlan

    dev = torch.device("cuda:0")
    if args.calibrate:  # a copy kernel of known size: reads 256 MiB, writes 256 MiB
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    n_layers = args.layers or {"c1": 64, "c2": 32, "c4": 4, "c5": 32}[args.workload]
    m = measure_decode(args.workload, n_layers, args.steps, args.warmup, args, dev)
    out = {
        "metric": METRIC,
        "value": round(m["us_per_step"], 3),
        "unit": "us/layer",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(m["us_per_step"] / 1e3, 6),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": m["config"],
        "timed_regions_us_per_step": m["regions"],
        "host_clock_us_per_step": round(m["us_per_step_host"], 3),
        "achieved_GBps": round(m["alg_bytes"] / (m["us_per_step"] * 1e-6) / 1e9, 1),
        "pct_of_hbm_peak": round(m["alg_bytes"] / (m["us_per_step"] * 1e-6) / 1e9 / HBM_PEAK_GBPS * 100, 2),
        "kernels_us": m["kernels_us"],
        "roofline": m["roofline"],
    }
    us_per_step, cfg, layers, plans, qs = m["us_per_step"], m["cfg"], m["layers"], m["plans"], m["qs"]
    sync = torch.cuda.synchronize
    if args.workload == "c2" and not args.no_extra:
        # the large-launch regime beside the headline: configuration 4's shape on a few layer caches
        del m
        try:
            x = measure_decode("c4", 3, 12, 3, args, dev)
            out["extra"] = {"workload": x["config"]["workload"], "layers_cycled": 3, "steps": 12, "warmup": 3,
                            "us_per_layer_step": round(x["us_per_step"], 2),
                            "timed_regions_us_per_step": x["regions"],
                            "achieved_GBps": round(x["alg_bytes"] / (x["us_per_step"] * 1e-6) / 1e9, 1),
                            "pct_of_hbm_peak": round(x["alg_bytes"] / (x["us_per_step"] * 1e-6) / 1e9 / HBM_PEAK_GBPS * 100, 2),
                            "kernels_us": x["kernels_us"], "roofline": x["roofline"]}
            del x
            torch.cuda.empty_cache()
        except torch.OutOfMemoryError as e:   # a smaller GPU: the headline stands on its own
            out["extra"] = {"skipped": f"configuration 4 does not fit: {e}"}

    if args.workload == "c2" and not args.no_extra:
        # the prompt side beside the headline: a short run of the causal prompt attention at the size of
        # `--workload prompt` (32768 tokens)
        try:
            out["extra_prompt"] = measure_prompt(32768, 4, 2)
        except (torch.OutOfMemoryError, RuntimeError) as e:
            out["extra_prompt"] = {"skipped": str(e)[:200]}

    if args.workload == "c5":
        # one generated token passes through every resident layer once
        out["decode_attention_only"] = {"layers": n_layers, "us_per_token_step": round(us_per_step * n_layers, 1),
                                        "tokens_per_s_attention_only": round(cfg["B"] / (us_per_step * n_layers * 1e-6), 1),
                                        "note": "the model's projections, MLP and prompt pass are outside this path"}
    if not args.no_cpu:
        base, (q_cpu, cache_cpu, ref) = cpu_baseline(args.workload, gpu_layer0=(qs[0], layers[0][1]))
        out["cpu_baseline"] = base
        # parity of layer 0 against the oracle on the same inputs (several batch rows: the first one)
        w, o = plans[0].run(qs[0])
        sync()
        nb = q_cpu.shape[0]
        out["parity_layer0"] = {
            "batch_rows_checked": nb,
            "attn_weights_max_abs": float((w[:nb].float().cpu() - ref[0].float()).abs().max()),
            "attn_output_max_abs": float((o[:nb].float().cpu() - ref[1].float()).abs().max()),
        }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
