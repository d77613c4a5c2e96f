#!/usr/bin/env python3
"""Benchmark of the hot path: decode attention over a Huffman-compressed KV cache on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2|cfg3|cfg4|cfg5] [--no-cpu-baseline]

A step is one decode-attention pass of one layer over the whole compressed cache, already resident in HBM:
fused decompress -> q.K^T, 1/sqrt(d) + softmax, fused decompress -> p.V, partial-sum reduce.  The printed value
is compressed-cache bytes (payload + block_infos + thread_infos + min + 2*scale, i.e. the denominator of the
reference's get_cr(), models/cache/kvcomp_encode.py:317-326, for K and V together) consumed per second.

One JSON line goes to stdout; progress goes to stderr.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E, published

# name -> shape and error bounds of the synthetic configurations
WORKLOADS = {
    # batch 1 Llama-2-7B layer, 4096 cached tokens
    "cfg2": dict(B=1, H=32, Hq=32, D=128, T=4096, eb_k=0.1, eb_v=0.2, dist="gauss",
                 desc="fused decode attention, Llama-2-7B layer: batch 1, 32 heads x 128, 4096 cached tokens, eb K 0.1 / V 0.2"),
    # batched GQA, Mistral-7B-shaped
    "cfg3": dict(B=16, H=8, Hq=32, D=128, T=8192, eb_k=0.1, eb_v=0.2, dist="gauss",
                 desc="batched GQA decode attention, Mistral-7B layer: batch 16, 32 q / 8 kv heads x 128, 8192 cached tokens, eb K 0.1 / V 0.2"),
    # long context, Phi-3-mini-shaped, heavy-tailed
    "cfg5": dict(B=4, H=32, Hq=32, D=96, T=32768, eb_k=0.1, eb_v=0.3, dist="laplace",
                 desc="long-context decode attention, Phi-3-mini layer: batch 4, 32 heads x 96, 32768 cached tokens, Laplace + 2% x50 outliers, eb K 0.1 / V 0.3"),
}
# every layer of a Llama-2-7B-shaped decoder, cache path only (see run_decode_loop)
WORKLOADS["cfg4"] = dict(layers=32, B=8, H=32, Hq=32, D=128, T=4096, eb_k=0.1, eb_v=0.2, dist="gauss",
                         desc="decode with a compressed KV cache in all 32 layers, Llama-2-7B shape: batch 8, 32 heads x 128, "
                              "4096-token prompt, one appended token per step, recompression every 64 (K) / 128 (V) tokens, "
                              "eb K 0.1 / V 0.2")
# the long-context configuration is the one the >= 70 % of HBM peak target is quoted on (32k context)
DEFAULT_WORKLOAD = "cfg5"


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def make_kv(cfg, device, seed_offset=0):
    """Synthetic K/V [T, B, H, D] fp16 from the CPU-seeded generators the tests use (tests/_synth.py): generated in
    fp32 on the host, cast to fp16, copied to the device, so that every run and the CPU oracle see the same bits."""
    from tests import _synth as S
    T, B, H, D = cfg["T"], cfg["B"], cfg["H"], cfg["D"]
    if cfg["dist"] == "gauss":
        k = S.synth_k(T, B, H, D, seed=S.SEED_K + 100 * seed_offset)
        v = S.synth_v(T, B, H, D, seed=S.SEED_V + 100 * seed_offset)
    else:
        k = S.synth_laplace(T, B, H, D, S.SEED_K + 100 * seed_offset)
        v = S.synth_laplace(T, B, H, D, S.SEED_V + 100 * seed_offset)
    return k.to(device), v.to(device)


def _sample_bytes(bi, nrows, cols, D, mask):
    import numpy as np
    tiles = nrows * cols
    payload = int(bi.view(np.uint32)[1::2][:tiles].astype(np.int64).sum())
    groups = tiles * D if mask == 0x1 else nrows
    return payload + tiles * 8 + tiles * 64 * 2 + groups * 3


def cpu_baseline(kctx, q, k_fp16, cfg, budget_s=10.0):
    """The reference's path restated on the host and timed on this machine's cores over bounded samples of the
    same workload.  `value` is the fused K algorithm (bit-serial tree walk, fp16 dequantize, dot; oracle/kvc_oracle.c:
    kvo_fused_k_from_stream) on all cores; `legs` adds the same on one thread, the reference's op-by-op PyTorch
    quantizer (utils/compute.py:93-106) on the CPU, and its pure-Python heapq Huffman coder (utils/huffman.py)."""
    import numpy as np
    import torch
    from oracle import oracle as O
    from kvcomp_amd.compute import dims_to_mask
    B, H, D, T = cfg["B"], cfg["H"], cfg["D"], cfg["T"]
    enc = kctx.encoded_data.cpu().numpy()
    bi = kctx.block_infos.cpu().numpy()
    ti = kctx.thread_infos.cpu().numpy()
    tree = kctx.decode_codebook.cpu().numpy()
    mn = kctx.quant_min_ints.cpu().numpy()
    sc = kctx.quant_scales.cpu().numpy()
    qh = q[:, ::cfg["Hq"] // H].contiguous().cpu().numpy()           # one query head per kv head
    mask = dims_to_mask(kctx.quant_dims)
    stride, rows, cols = B * H * D, T // 64, B * H
    cores = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(16, os.cpu_count() or 1)

    def fused_leg(threads, budget):
        O.lib().kvo_set_threads(threads)

        def run(nrows):
            t0 = time.perf_counter()
            O.fused_k_from_stream(enc, bi, ti, tree, mn, sc, qh, nrows * 64, stride, vec_len=D, mask=mask)
            return time.perf_counter() - t0

        probe = max(1, min(rows, 2))
        dt = run(probe)
        nrows = int(max(probe, min(rows, probe * budget / max(dt, 1e-6))))
        reps, total = 0, 0.0
        while total < budget and reps < 200:          # repeat the bounded sample until ~budget seconds are timed
            total += run(nrows)
            reps += 1
        return reps * _sample_bytes(bi, nrows, cols, D, mask) / total / 1e9, nrows, reps, total

    gbs, nrows, reps, total = fused_leg(cores, budget_s)
    out = {"value": round(gbs, 4), "unit": "GB/s", "cores": cores, "kind": "port",
           "sample": "fused K (bit-serial tree-walk decode + fp16 dequant + dot, OpenMP over tiles) over the first %d of "
                     "%d tokens of the same compressed K stream, %d passes, %.1f s" % (nrows * 64, T, reps, total)}
    legs = {}
    g1, n1, r1, t1 = fused_leg(1, 4.0)
    legs["fused_k_single_thread"] = {"value": round(g1, 4), "unit": "GB/s compressed", "cores": 1,
                                     "sample": "first %d tokens, %d passes, %.1f s" % (n1 * 64, r1, t1)}
    O.lib().kvo_set_threads(cores)
    # the reference quantizer, one fp16 PyTorch op after the other (utils/compute.py:93-106), per-channel K groups
    xs = k_fp16[:min(T, 2048)].cpu().reshape(-1, 64, B, H, D)
    torch.set_num_threads(cores)
    t0, n = time.perf_counter(), 0
    while time.perf_counter() - t0 < 4.0:
        mx, mi = xs.amax(dim=1, keepdim=True), xs.amin(dim=1, keepdim=True)
        scale = (mx - mi) * cfg["eb_k"]
        sym = (xs / scale).round() - (mi / scale).round()
        n += 1
    dt = time.perf_counter() - t0
    legs["pytorch_cpu_quantizer"] = {"value": round(n * xs.numel() * 2 / dt / 1e9, 4), "unit": "GB/s fp16 in", "cores": cores,
                                     "sample": "max/min/sub/mul/div/round/sub as separate fp16 CPU ops on the first %d tokens of K, "
                                               "%d passes, %.1f s" % (xs.shape[0] * 64, n, dt)}
    del sym
    # the reference's whole-tensor Huffman coder (heapq tree + per-symbol string concatenation), 64 Ki symbols
    syms = kctx.get_decode_quant_ints()[0].reshape(-1)[:65536].cpu().numpy()
    t0 = time.perf_counter()
    book = O.py_huffman_codebook(syms)
    bits = O.py_bits(syms, book)
    dt = time.perf_counter() - t0
    legs["python_heapq_huffman"] = {"value": round(syms.size / dt / 1e9, 6), "unit": "GB/s symbols in", "cores": 1,
                                    "sample": "65536 symbols of K, %d bits out, %.1f ms (pure Python: not extrapolated)" % (bits.size, dt * 1e3)}
    out["legs"] = legs
    return out


def codec_rates(kctx, vctx, k, v, cfg):
    """Huffman encode / decode throughput of the non-fused kernels, on the same tensors (GB/s)."""
    import torch
    from kvcomp_amd import kvcomp_cuda as m
    from kvcomp_amd.compute import quant
    out = {}
    for name, ctx, x in (("k", kctx, k), ("v", vctx, v)):
        blocked = x.reshape(-1, ctx.block_size, ctx.batch_size, ctx.head_num, ctx.head_dim)
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
        ev[0].record()
        sym, _, _ = quant(blocked, ctx.quant_dims, ctx.quant_scale_rel)
        ev[1].record()
        sizes = m.calculate_buffer_size(sym, ctx.is_k, ctx.head_num, ctx.head_dim)
        bufs = ctx._scratch(sizes)
        fn = m.k_entropy_encode_cuda_export if ctx.is_k else m.v_entropy_encode_cuda_export
        ev[2].record()
        fn(sym, ctx.encode_codebook, bufs[0], bufs[1], bufs[2], bufs[3], 0, ctx.head_num, ctx.head_dim)
        ev[3].record()
        torch.cuda.synchronize()
        _, dec_ms = ctx.get_decode_quant_ints()
        _, dec_ms = ctx.get_decode_quant_ints()
        _, deq_ms = ctx.get_only_compressed()               # decode + dequantize in one kernel: fp16 out
        _, deq_ms = ctx.get_only_compressed()
        n = sym.numel()
        del sym
        # the same store as one fused call straight from fp16 (codebook known): quantize + encode, no symbol tensor
        from kvcomp_amd.compute import dims_to_mask, mask_keepdim_shape
        mask = dims_to_mask(ctx.quant_dims)
        fused_ms = None
        if m.store_fused_supported(ctx.is_k, mask, ctx.batch_size, ctx.head_num, ctx.head_dim):
            gshape = mask_keepdim_shape(tuple(blocked.shape), mask)
            mn = torch.empty(gshape, dtype=torch.int8, device=x.device)
            sc = torch.empty(gshape, dtype=torch.float16, device=x.device)
            for _ in range(2):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                m.store_fused(ctx.is_k, x, mask, ctx.quant_scale_rel, ctx.encode_codebook, mn, sc, bufs[0], bufs[1], bufs[2],
                              bufs[3], 0)
                e1.record()
                torch.cuda.synchronize()
                fused_ms = e0.elapsed_time(e1)
            del mn, sc
        out[name] = {"store_fused_GBs_fp16_in": round(2 * n / fused_ms / 1e6, 1) if fused_ms else None,
                     "quantize_GBs_fp16_in": round(2 * n / ev[0].elapsed_time(ev[1]) / 1e6, 1),
                     "huffman_encode_GBs_fp16_equiv": round(2 * n / ev[2].elapsed_time(ev[3]) / 1e6, 1),
                     "huffman_encode_GBs_symbols_in": round(n / ev[2].elapsed_time(ev[3]) / 1e6, 1),
                     "huffman_decode_GBs_symbols_out": round(n / dec_ms / 1e6, 1),
                     "decode_dequant_GBs_fp16_out": round(2 * n / deq_ms / 1e6, 1)}
    return out


def kernel_sources_digest():
    """Digest of the kernel sources: measured counter figures are only quoted for the sources they were taken on."""
    import hashlib
    h = hashlib.sha256()
    d = os.path.join(ROOT, "kvcomp_amd", "csrc")
    for name in sorted(os.listdir(d)):
        if name.endswith((".hip", ".h")):
            with open(os.path.join(d, name), "rb") as f:
                h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()[:16]


def measured_traffic(workload, kernel):
    """HBM bytes per launch of `kernel` from profiles/traffic.json: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per
    dispatch), each scaled by what the same counter reads for the 256 MiB kvc_calibration_copy_kernel of the same run.
    None when the file has no figure for this kernel, or when it was measured on other kernel sources than these."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            t = json.load(f)
    except (OSError, ValueError):
        return None
    if t.get("kernel_sources_digest") != kernel_sources_digest():
        return None
    return t.get("bytes_per_launch", {}).get(workload, {}).get(kernel)


def check_layer_attention(attn, q, tokens):
    """One layer's decode attention against fp32 attention over the dequantized cache (compressed part + fp16 tail, as
    KVCompCtx.get() returns it), a batch entry at a time; returns the largest error relative to max|reference| and
    raises beyond the 1e-3 this path is held to."""
    import torch
    kctx, vctx = attn.k, attn.v
    out = attn.attend(q)
    kd, vd = kctx.get()[0], vctx.get()[0]
    assert kd.shape[0] == vd.shape[0] == tokens
    B, Hq, D = q.shape
    rep = Hq // kctx.head_num
    worst = 0.0
    for b in range(B):
        kb, vb = kd[:, b].float().repeat_interleave(rep, dim=1), vd[:, b].float().repeat_interleave(rep, dim=1)
        s = torch.einsum("thd,hd->ht", kb, q[b].float()) / D ** 0.5
        ref = torch.einsum("ht,thd->hd", torch.softmax(s, dim=-1), vb)
        worst = max(worst, float((out[b] - ref).abs().max() / ref.abs().max()))
    assert worst <= 1e-3, "decode attention differs from fp32 attention over the dequantized cache by %.2e" % worst
    return worst


def run_decode_loop(args, emit=True):
    """cfg4 without the model around it: every layer of a Llama-2-7B-shaped stack keeps a compressed K and V cache;
    a step appends one new token per sequence to every layer (compressing the 64- / 128-token blocks that leave
    the uncompressed tails) and runs decode attention over the whole cache of that layer.  Projections, MLPs and
    sampling are not part of this path and are not run; keys, values and queries are random."""
    import torch
    from kvcomp_amd.ctx import KVCompCtx, KVCompCacheConfig, KVCompCacheConfigStatic, QuantMode
    from kvcomp_amd import attention as A
    cfg = WORKLOADS["cfg4"]
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    L, B, H, Hq, D, T = cfg["layers"], cfg["B"], cfg["H"], cfg["Hq"], cfg["D"], cfg["T"]
    KVCompCacheConfigStatic.config = KVCompCacheConfig("cfg4", QuantMode.ChannelQuant, QuantMode.TokenQuant,
                                                       64, 128, 64, 128, cfg["eb_k"], cfg["eb_v"])
    log("[bench] %s" % cfg["desc"])
    layers = []
    t_prefill = 0.0                              # the stores alone: the inputs are generated on the host, layer by layer
    for l in range(L):
        k, v = make_kv(cfg, dev, seed_offset=l)
        kctx, vctx = KVCompCtx(True, B, H, D, cfg["eb_k"]), KVCompCtx(False, B, H, D, cfg["eb_v"])
        for c in (kctx, vctx):                   # as the model-facing caches set their contexts up
            c.codebook_smoothing = True          # later tokens may quantize to symbols the prompt never produced
            c.async_store = not args.sync_store  # blocks that leave the tail are encoded without waiting for the device
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        kctx.store(k, want_symbols=False)
        vctx.store(v, want_symbols=False)
        torch.cuda.synchronize()
        t_prefill += time.perf_counter() - t0
        layers.append((kctx, vctx, A.CompressedAttention(kctx, vctx)))
        del k, v
    g = torch.Generator(device=dev).manual_seed(1236)
    new_k = torch.randn(L, 1, B, H, D, generator=g, device=dev).to(torch.float16)
    new_v = torch.randn(L, 1, B, H, D, generator=g, device=dev).to(torch.float16)
    q = torch.randn(L, B, Hq, D, generator=g, device=dev).to(torch.float16)
    out = torch.empty(B, Hq, D, dtype=torch.float32, device=dev)

    def step():
        for l, (kctx, vctx, attn) in enumerate(layers):
            kctx.store(new_k[l], want_symbols=False)
            vctx.store(new_v[l], want_symbols=False)
            attn.attend(q[l], out=out)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert torch.isfinite(out).all()
    # after the timed steps: two layers' operators against fp32 attention over what their caches hold now
    check_err = max(check_layer_attention(layers[l][2], q[l], layers[l][0].ctx_len) for l in (0, L - 1))
    log("[bench] cfg4 cache loop checked against fp32 attention over the dequantized cache (layers 0 and %d): max error %.1e" % (L - 1, check_err))
    comp = sum(k.compressed_bytes() + v.compressed_bytes() for k, v, _ in layers)
    tails = sum((k.buffer.numel() + v.buffer.numel()) * 2 for k, v, _ in layers)
    tokens = layers[0][0].ctx_len
    raw = 2 * 2 * L * tokens * B * H * D
    result = {
        "metric": "decode tokens/s with a compressed KV cache in every layer (cache append + attention only)",
        "value": round(B * args.steps / dt, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(dt / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8 symbols, fp32 accumulate", "data": "synthetic",
        "config": {"workload": "cfg4: %s" % cfg["desc"], "layers": L, "context_at_end": tokens,
                   "cache_bytes": {"compressed": comp, "fp16_tails": tails, "fp16_equivalent": raw},
                   "compression_ratio_whole_cache": round(raw / (comp + tails), 3),
                   "compression_ratio_compressed_part": {"k": round(layers[0][0].get_cr(), 3), "v": round(layers[0][1].get_cr(), 3)},
                   "prefill_compress_s": round(t_prefill, 3), "check_max_error": check_err,
                   "not_run": "projections, MLP, norms, sampling (outside this path)"},
        "roofline": None, "cpu_baseline": None,
    }
    if emit:
        print(json.dumps(result), flush=True)
    del layers
    torch.cuda.empty_cache()
    return result


def graph_replay_ms(attns, q, out, steps, warmup, name):
    """ms per step of the attention call recorded in HIP graphs and replayed: one graph per copy of the cache, replayed
    in turn, so that the streams come from HBM as they do in the eager figure (a single small cache would stay in the
    last-level cache).  The library call allocates nothing and waits for nothing, so it is recorded as it is; every
    graph's first replay is checked against the eager call."""
    import torch
    side = torch.cuda.Stream()
    graphs = []
    with torch.cuda.stream(side):
        for a in attns:
            a.attend(q, out=out)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=side):
                a.attend(q, out=out)
            graphs.append(g)
    torch.cuda.synchronize()
    for a, g in zip(attns, graphs):
        eager = a.attend(q).clone()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), "%s: graph replay differs from the eager call" % name
    n = len(graphs)
    for i in range(warmup):
        graphs[i % n].replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        graphs[i % n].replay()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    del graphs
    return ms


def quick_attention(name, steps=50, warmup=10):
    """One of the smaller configurations, measured the short way for the default run's `config.other_configs`: build the
    compressed cache, check one result against fp32 attention over the dequantized cache, time `steps` decode-attention
    passes (default arithmetic) over copies of the cache that together exceed the last-level cache."""
    import copy
    import torch
    from kvcomp_amd.ctx import KVCompCtx, KVCompCacheConfig, KVCompCacheConfigStatic, QuantMode
    from kvcomp_amd import attention as A
    cfg = WORKLOADS[name]
    dev = torch.device("cuda:0")
    B, H, Hq, D, T = cfg["B"], cfg["H"], cfg["Hq"], cfg["D"], cfg["T"]
    KVCompCacheConfigStatic.config = KVCompCacheConfig(name, QuantMode.ChannelQuant, QuantMode.TokenQuant, 64, 128, 64, 128,
                                                       cfg["eb_k"], cfg["eb_v"])
    k, v = make_kv(cfg, dev)
    kctx, vctx = KVCompCtx(True, B, H, D, cfg["eb_k"]), KVCompCtx(False, B, H, D, cfg["eb_v"])
    kctx.store(k, want_symbols=False)
    vctx.store(v, want_symbols=False)
    rates = codec_rates(kctx, vctx, k, v, cfg)           # encode / decode rates of the same prompt cache (GB/s)
    del k, v
    g = torch.Generator().manual_seed(1236)
    q = torch.randn(B, Hq, D, generator=g, dtype=torch.float32).to(torch.float16).to(dev)
    kb, vb = kctx.compressed_bytes(), vctx.compressed_bytes()
    n = max(3, min(32, -(-600_000_000 // (kb + vb))))
    attns = [A.CompressedAttention(kctx, vctx)] + [A.CompressedAttention(copy.deepcopy(kctx), copy.deepcopy(vctx)) for _ in range(n - 1)]
    out = torch.empty(B, Hq, D, dtype=torch.float32, device=dev)
    attns[0].attend(q, out=out)
    rep = Hq // H
    kd, vd = kctx.get_only_compressed()[0][:, 0, 0].float(), vctx.get_only_compressed()[0][:, 0, 0].float()   # batch 0, KV head 0
    sc = torch.einsum("td,rd->rt", kd, q[0, :rep].float()) / D ** 0.5
    ref = torch.einsum("td,rt->rd", vd, torch.softmax(sc, dim=-1))
    err = float((out[0, :rep] - ref).abs().max() / ref.abs().max())
    assert err <= 1e-3, "%s: attention differs from fp32 attention over the dequantized cache by %.2e" % (name, err)
    for i in range(warmup):
        attns[i % n].attend(q, out=out)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        attns[i % n].attend(q, out=out)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    k_ms = v_ms = 0.0
    for i in range(steps):
        kms = []
        attns[i % n].attend(q, out=out, kernel_ms=kms)
        k_ms += kms[0] / steps
        v_ms += kms[1] / steps
    # the same step captured in HIP graphs and replayed (where the step is launch-bound, this is what counts)
    graph_ms = graph_replay_ms(attns, q, out, steps, warmup, name)
    res = {"workload": cfg["desc"], "ms_per_step": round(ms, 4), "GBs": round((kb + vb) / (ms * 1e-3) / 1e9, 1),
           "pct_hbm_peak": round(100 * (kb + vb) / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 2),
           "graph_replay_ms_per_step": round(graph_ms, 4), "codec": rates,
           "kernels_ms": {"fused_k": round(k_ms, 4), "fused_v": round(v_ms, 4)}, "compressed_bytes": {"k": kb, "v": vb},
           "compression_ratio": {"k": round(kctx.get_cr(), 3), "v": round(vctx.get_cr(), 3)},
           "k_max_code_bits": kctx.max_code_bits, "v_max_code_bits": vctx.max_code_bits,
           "cache_copies_cycled": n, "steps": steps, "check_max_error": err}
    log("[bench] %s: step %.3f ms (%.0f GB/s of compressed bytes; as a replayed graph %.3f ms), fused K %.3f ms, fused V %.3f ms; "
        "fused store K %.0f / V %.0f GB/s of fp16 in" % (name, ms, res["GBs"], graph_ms, k_ms, v_ms,
                                                        rates["k"]["store_fused_GBs_fp16_in"] or 0, rates["v"]["store_fused_GBs_fp16_in"] or 0))
    del attns, kctx, vctx
    torch.cuda.empty_cache()
    return res


def other_configs(args):
    """The configurations besides the default one, each measured briefly in the same process."""
    import types
    res = {}
    for name in ("cfg2", "cfg3"):
        res[name] = quick_attention(name)
    loop = run_decode_loop(types.SimpleNamespace(steps=20, warmup=5, sync_store=False), emit=False)
    res["cfg4_cache_loop"] = {"workload": loop["config"]["workload"], "ms_per_step": loop["ms_per_step"], "tokens_per_s": loop["value"],
                              "steps": loop["steps"], "compression_ratio_whole_cache": loop["config"]["compression_ratio_whole_cache"],
                              "prefill_compress_s": loop["config"]["prefill_compress_s"], "check_max_error": loop["config"]["check_max_error"],
                              "not_run": loop["config"]["not_run"]}
    log("[bench] cfg4 cache loop: %.2f ms per step, %.0f tokens/s" % (loop["ms_per_step"], loop["value"]))
    # cfg4 with the model around the cache (random weights), and the same model on transformers' dense fp16 cache
    try:
        import transformers  # noqa: F401
    except ImportError:
        res["cfg4_model"] = None
        return res
    model = {}
    for key, dense in (("compressed_cache", False), ("dense_fp16_cache", True)):
        r = run_model_decode(types.SimpleNamespace(model_layers=32, new_tokens=64, warmup=5, dense_cache=dense), emit=False)
        model[key] = {"tokens_per_s": r["value"], "ms_per_step": r["ms_per_step"], "steps": r["steps"],
                      "prefill_s": r["config"]["prefill_s"], "cache_bytes_held": r["config"]["cache_bytes_held"],
                      "compression_ratio_whole_cache": r["config"]["compression_ratio_whole_cache"],
                      "check_max_error": r["config"]["check_max_error"], "attention": r["config"]["attention"]}
        log("[bench] cfg4 model, %s: %.2f ms per step, %.0f tokens/s" % (key.replace("_", " "), r["ms_per_step"], r["value"]))
    model["workload"] = "Llama-2-7B architecture (stock transformers code, random fp16 weights), 32 layers, batch 8, 4096-token random prompt, 64 greedy tokens"
    res["cfg4_model"] = model
    return res


def run_model_decode(args, emit=True):
    """cfg4 as the headline configuration list words it: the Llama-2-7B architecture with random-init fp16 weights (stock `transformers`
    modelling code), a compressed KV cache in every layer, batch 8, a 4096-token random prompt and greedy generation;
    single-token steps attend on the compressed form through the "kvcomp" attention implementation.  Tokens are random,
    so the text means nothing; the arithmetic and the memory traffic are those of the real model."""
    import torch
    from transformers import LlamaConfig, LlamaForCausalLM
    from kvcomp_amd import hf_adapter as HA
    from kvcomp_amd.ctx import KVCompCacheConfig, KVCompCacheConfigStatic, QuantMode
    cfg = WORKLOADS["cfg4"]
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    L = args.model_layers
    B, H, D, T = cfg["B"], cfg["H"], cfg["D"], cfg["T"]
    KVCompCacheConfigStatic.config = KVCompCacheConfig("cfg4", QuantMode.ChannelQuant, QuantMode.TokenQuant,
                                                       64, 128, 64, 128, cfg["eb_k"], cfg["eb_v"])
    log("[bench] Llama-2-7B architecture, %d layers, random fp16 weights, batch %d, %d-token prompt, %d generated tokens"
        % (L, B, T, args.new_tokens))
    mcfg = LlamaConfig(vocab_size=32000, hidden_size=H * D, intermediate_size=11008, num_hidden_layers=L,
                       num_attention_heads=H, num_key_value_heads=H, max_position_embeddings=T + args.new_tokens + 64,
                       attn_implementation="sdpa")
    torch.manual_seed(1240)
    old_dtype = torch.get_default_dtype()
    torch.set_default_dtype(torch.float16)
    try:
        with torch.device(dev):
            model = LlamaForCausalLM(mcfg).eval()
    finally:
        torch.set_default_dtype(old_dtype)
    g = torch.Generator().manual_seed(1239)
    ids = torch.randint(0, 32000, (B, T), generator=g).to(dev)
    if args.dense_cache:                     # comparison run: transformers' own fp16 cache and attention
        from transformers import DynamicCache
        cache = DynamicCache()
    else:
        model.set_attn_implementation(HA.register_kvcomp_attention())
        cache = HA.KVCompHFCache(attend_compressed=True)
    with torch.no_grad():
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = model(ids, past_key_values=cache, use_cache=True, logits_to_keep=1).logits
        nxt = logits[:, -1].argmax(-1, keepdim=True)
        torch.cuda.synchronize()
        t_prefill = time.perf_counter() - t0
        for _ in range(args.warmup):
            nxt = model(nxt, past_key_values=cache, use_cache=True).logits[:, -1].argmax(-1, keepdim=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.new_tokens):
            nxt = model(nxt, past_key_values=cache, use_cache=True).logits[:, -1].argmax(-1, keepdim=True)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
    check_err = None
    if not args.dense_cache:
        # the first and the last layer's streams as generation left them: the operator the model attended with against
        # fp32 attention over the dequantized cache, with a fresh random query
        from kvcomp_amd.attention import CompressedAttention
        gq = torch.Generator().manual_seed(1236)
        qs = torch.randn(B, H, D, generator=gq, dtype=torch.float32).to(torch.float16).to(dev)
        check_err = max(check_layer_attention(CompressedAttention(cache.layers[l].k_ctx, cache.layers[l].v_ctx), qs,
                                              cache.get_seq_length()) for l in (0, L - 1))
        log("[bench] cfg4 model: layers 0 and %d checked against fp32 attention over the dequantized cache: max error %.1e" % (L - 1, check_err))
    result = {
        "metric": "decode tokens/s, Llama-2-7B architecture (random weights) with a compressed KV cache in every layer",
        "value": round(B * args.new_tokens / dt, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.new_tokens,
        "warmup": args.warmup, "ms_per_step": round(dt / args.new_tokens * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "fp16 model, u8 symbols, fp32 accumulate in attention",
        "data": "synthetic",
        "config": {"workload": "cfg4 with the model: %d layers, batch %d, %d-token prompt, greedy decoding" % (L, B, T),
                   "context_at_end": cache.get_seq_length(),
                   "compression_ratio_whole_cache": None if args.dense_cache else round(cache.compression_ratio(), 3),
                   "cache_bytes_held": (2 * 2 * L * cache.get_seq_length() * B * H * D if args.dense_cache
                                        else cache.compressed_bytes()),
                   "prefill_s": round(t_prefill, 3), "check_max_error": check_err,
                   "attention": ("transformers DynamicCache (dense fp16) and stock SDPA: the comparison run" if args.dense_cache else
                                 "single-token steps: kvc_attention_decode on the compressed streams; prompt: stock SDPA")},
        "roofline": None, "cpu_baseline": None,
    }
    if emit:
        print(json.dumps(result), flush=True)
    del model, cache, logits, nxt
    torch.cuda.empty_cache()
    return result


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default=DEFAULT_WORKLOAD, choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--eb-k", type=float, default=None, help="override the K error bound of the workload (cfg5 sweeps 0.05 / 0.1 / 0.2)")
    ap.add_argument("--no-unrounded", action="store_true",
                    help="skip the extra pass in unrounded mode (keeps a kernel trace of this run to one variant per kernel)")
    ap.add_argument("--settle-seconds", type=float, default=0.5,
                    help="untimed run of the operator before warm-up, so the timed steps see the sustained clock")
    ap.add_argument("--no-sweep", action="store_true", help="cfg5: skip the sweep over K's error bound")
    ap.add_argument("--sync-store", action="store_true",
                    help="cfg4: wait for the device after every encode (the reference's behaviour) instead of queuing it")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="default workload: skip the short measurements of cfg2, cfg3 and the cfg4 cache loop (config.other_configs)")
    ap.add_argument("--no-graph", action="store_true", help="skip the replay of the step as a captured HIP graph")
    ap.add_argument("--model-layers", type=int, default=0,
                    help="cfg4 only: run the Llama-2-7B architecture itself (random weights) with this many layers (32 = "
                         "the whole model) instead of the cache-and-attention loop")
    ap.add_argument("--dense-cache", action="store_true",
                    help="cfg4 with --model-layers: use transformers' dense fp16 cache and attention instead (comparison run)")
    ap.add_argument("--new-tokens", type=int, default=256, help="cfg4 with --model-layers: tokens generated after the prompt")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch one plain 256 MiB device copy (kvc_calibration_copy_kernel), the yardstick "
                         "for FETCH_SIZE / WRITE_SIZE when this command runs under rocprofv3 --pmc")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py measures one GPU: this path shards by KV head or batch with no exchange, and no run here "
            "uses a second GPU (--gpus %d refused)" % args.gpus)
        sys.exit(2)

    import copy
    import torch
    from kvcomp_amd import _lib
    from kvcomp_amd.ctx import KVCompCtx, KVCompCacheConfig, KVCompCacheConfigStatic, QuantMode
    from kvcomp_amd import attention as A

    if args.workload == "cfg4":
        return run_model_decode(args) if args.model_layers > 0 else run_decode_loop(args)
    cfg = dict(WORKLOADS[args.workload])
    if args.eb_k is not None:
        cfg["desc"] = cfg["desc"].replace("eb K %g" % cfg["eb_k"], "eb K %g" % args.eb_k)
        cfg["eb_k"] = args.eb_k
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    B, H, Hq, D, T = cfg["B"], cfg["H"], cfg["Hq"], cfg["D"], cfg["T"]
    rep = Hq // H
    KVCompCacheConfigStatic.config = KVCompCacheConfig(args.workload, QuantMode.ChannelQuant, QuantMode.TokenQuant,
                                                       64, 128, 64, 128, cfg["eb_k"], cfg["eb_v"])
    log("[bench] %s" % cfg["desc"])
    t0 = time.perf_counter()
    k, v = make_kv(cfg, dev)
    log("[bench] inputs generated on the host (seeded) in %.1f s" % (time.perf_counter() - t0))
    # the first store of a stream (quantize, histogram, codebook and decode tables on the device, encode), timed on
    # a second pair of contexts so that the caching allocator has the buffers at hand (a first cudaMalloc of several
    # hundred MB costs more than the work)
    for _ in range(2):
        kctx, vctx = KVCompCtx(True, B, H, D, cfg["eb_k"]), KVCompCtx(False, B, H, D, cfg["eb_v"])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        kctx.store(k, want_symbols=False)
        vctx.store(v, want_symbols=False)
        torch.cuda.synchronize()
        t_store = time.perf_counter() - t0
    rates = codec_rates(kctx, vctx, k, v, cfg)
    assert kctx.compressed_ctx_len == T and vctx.compressed_ctx_len == T
    kb, vb = kctx.compressed_bytes(), vctx.compressed_bytes()
    numel = T * B * H * D
    log("[bench] compressed: K %.1f MB (CR %.2f, %.2f bits/sym)  V %.1f MB (CR %.2f, %.2f bits/sym); first store "
        "(incl. codebook) %.1f ms" % (kb / 1e6, kctx.get_cr(), 8 * kctx.encoded_data.numel() / numel, vb / 1e6,
                                      vctx.get_cr(), 8 * vctx.encoded_data.numel() / numel, t_store * 1e3))

    g = torch.Generator().manual_seed(1236)
    q = torch.randn(B, Hq, D, generator=g, dtype=torch.float32).to(torch.float16).to(dev)

    # Several copies of the compressed cache, visited in turn, so that no step finds its stream in the 256 MiB
    # last-level cache left there by the step before: the copies together hold at least 600 MB.
    def cache_copies(kc, vc):
        n = max(3, min(32, -(-600_000_000 // (kc.compressed_bytes() + vc.compressed_bytes()))))
        return [A.CompressedAttention(kc, vc)] + [A.CompressedAttention(copy.deepcopy(kc), copy.deepcopy(vc)) for _ in range(n - 1)]

    def time_steps(attns, steps, warmup):
        """ms per step over `steps` steps between two synchronisations (the contract's figure), the per-step times
        from events on the launch stream, and the mean durations of the two fused kernels from a second pass in
        which the library brackets them by events of its own (that makes every call wait, so it is a pass apart)."""
        out = torch.empty(B, Hq, D, dtype=torch.float32, device=dev)
        n = len(attns)
        for i in range(warmup):
            attns[i % n].attend(q, out=out)
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            ev[i][0].record()
            attns[i % n].attend(q, out=out)
            ev[i][1].record()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) / steps * 1e3
        per = sorted(a.elapsed_time(b) for a, b in ev)
        pick = lambda f: per[min(len(per) - 1, int(f * len(per)))]
        k_ms = v_ms = 0.0
        for i in range(steps):
            kms = []
            attns[i % n].attend(q, out=out, kernel_ms=kms)
            k_ms += kms[0] / steps
            v_ms += kms[1] / steps
        assert torch.isfinite(out).all()
        return {"ms_per_step": ms, "event_ms": {"median": round(pick(0.5), 4), "p10": round(pick(0.1), 4), "p90": round(pick(0.9), 4)},
                "k_ms": k_ms, "v_ms": v_ms, "out": out}

    if args.copy_calibration:
        import ctypes
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        _lib.check(_lib.lib().kvc_calibration_copy(ctypes.c_void_p(dst.data_ptr()), ctypes.c_void_p(src.data_ptr()),
                                                   src.numel(), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
        torch.cuda.synchronize()
        del src, dst

    attns = cache_copies(kctx, vctx)
    n_copies = len(attns)
    # Before anything is timed: the operator against fp32 attention over the fp16 cache the reference's dequantizer
    # gives (models/cache/kvcomp_encode.py:146), on one (batch, head) slice of this very cache, within 1e-3.
    _lib.set_option("fused_rounded", 1)          # the headline is this mode, whatever the environment preset
    check = attns[0].attend(q)
    kd = kctx.get_only_compressed()[0][:, 0, 0].float()
    vd = vctx.get_only_compressed()[0][:, 0, 0].float()
    for r in range(rep):
        sref = torch.softmax((kd @ q[0, r].float()) / D ** 0.5, dim=0)
        oref = sref @ vd
        err = float((check[0, r] - oref).abs().max() / oref.abs().max())
        assert err <= 1e-3, "decode attention differs from fp32 attention over the dequantized cache by %.2e" % err
    del kd, vd
    log("[bench] checked against fp32 attention over the dequantized cache (batch 0, KV head 0): max error %.1e of max|out|" % err)

    # The card idles at a low clock while the host prepares inputs and takes some hundred milliseconds of work to
    # reach its sustained one (the same pass, timed later in this run, was 8 - 10 % faster than when timed first):
    # the operator runs untimed for a moment, then come the --warmup steps and the timed ones.
    t_end = time.perf_counter() + args.settle_seconds
    while time.perf_counter() < t_end:
        for a in attns:
            a.attend(q)
        torch.cuda.synchronize()
    res = time_steps(attns, args.steps, args.warmup)
    ms_per_step, k_ms, v_ms = res["ms_per_step"], res["k_ms"], res["v_ms"]
    log("[bench] step %.3f ms (events: median %.3f, p10 %.3f, p90 %.3f) over %d copies of the cache; fused K kernel %.3f ms "
        "(%.1f GB/s compressed), fused V kernel %.3f ms (%.1f GB/s compressed)"
        % (ms_per_step, res["event_ms"]["median"], res["event_ms"]["p10"], res["event_ms"]["p90"], len(attns), k_ms,
           kb / k_ms / 1e6, v_ms, vb / v_ms / 1e6))
    # the same pass with the dequantized values left unrounded (fp32 products; not the reference's cache values)
    unrounded = None
    if not args.no_unrounded:
        was = _lib.set_option("fused_rounded", 0)
        try:
            u = time_steps(attns, args.steps, args.warmup)
        finally:
            _lib.set_option("fused_rounded", was)
        unrounded = {"ms_per_step": round(u["ms_per_step"], 4), "GBs": round((kb + vb) / (u["ms_per_step"] * 1e-3) / 1e9, 1),
                     "event_ms": u["event_ms"], "kernels_ms": {"fused_k": round(u["k_ms"], 4), "fused_v": round(u["v_ms"], 4)},
                     "max_difference_from_default": float((u["out"] - res["out"]).abs().max() / res["out"].abs().max())}
        log("[bench] unrounded mode: step %.3f ms; fused K %.3f ms, fused V %.3f ms" % (u["ms_per_step"], u["k_ms"], u["v_ms"]))

    # the same step captured once in a HIP graph and replayed (what a serving loop does with a launch-bound step:
    # the library call allocates nothing and waits for nothing, so it can be recorded as it is)
    graph_ms = None
    if not args.no_graph:
        out = torch.empty(B, Hq, D, dtype=torch.float32, device=dev)
        graph_ms = graph_replay_ms(attns, q, out, args.steps, args.warmup, args.workload)
        log("[bench] one step as a HIP graph, replayed (a graph per copy of the cache, in turn): %.3f ms" % graph_ms)

    # cfg5 sweeps K's error bound (V fixed): one entry per bound, the same step on a cache compressed with it
    sweep = None
    if args.workload == "cfg5" and args.eb_k is None and not args.no_sweep:
        sweep = []
        for eb in (0.05, 0.1, 0.2):
            at = None                                  # the previous bound's copies are released first
            if eb == cfg["eb_k"]:
                kc, at = kctx, attns
            else:
                kc = KVCompCtx(True, B, H, D, eb)
                kc.store(k, want_symbols=False)
                at = cache_copies(kc, vctx)
            r = time_steps(at, args.steps, args.warmup)
            bits = kc.max_code_bits
            loop = ("matrix-core kernel, two symbols per look-up" if 2 * bits <= 8 else
                    "matrix-core kernel, one symbol per look-up, %d per refill" % (16 if bits <= 3 else 12 if bits <= 5 else 8)
                    if bits <= 7 else "fp32-FMA kernel, one symbol per look-up" if bits <= 10 else
                    "fp32-FMA kernel, one symbol per refill (codes beyond the table index)")
            sweep.append({"eb_k": eb, "ms_per_step": round(r["ms_per_step"], 4),
                          "GBs": round((kc.compressed_bytes() + vb) / (r["ms_per_step"] * 1e-3) / 1e9, 1),
                          "fused_k_ms": round(r["k_ms"], 4), "k_compressed_bytes": kc.compressed_bytes(),
                          "k_bits_per_symbol": round(8 * kc.encoded_data.numel() / numel, 3), "k_max_code_bits": bits,
                          "k_decode_loop": loop})
            log("[bench] eb K %.2f: step %.3f ms, fused K %.3f ms, %.2f bits/sym, codes up to %d bits (%s)"
                % (eb, r["ms_per_step"], r["k_ms"], sweep[-1]["k_bits_per_symbol"], bits, loop))
    del k, v

    # template arguments: query heads per KV head, then 0 = K tile, 3 / 4 = V tile with the softmax on the fly
    # (4: head_dim is not a multiple of 64, tiles may straddle two heads), then rounded mode
    v_kind = 3 if D % 64 == 0 else 4
    mfma = kctx.max_code_bits <= 7, vctx.max_code_bits <= 7
    name = lambda kind, m: ("kvc_fused_mfma_kernel<%d, %d, true>" % (rep, kind)) if m else ("kvc_fused_kernel<%d, %d>" % (rep, kind))
    dom, dom_ms, dom_bytes = ((name(0, mfma[0]), k_ms, kb) if k_ms >= v_ms else (name(v_kind, mfma[1]), v_ms, vb))
    achieved = dom_bytes / dom_ms / 1e6
    value = (kb + vb) / (ms_per_step * 1e-3) / 1e9
    result = {
        "metric": "fused decompress-matvec GB/s (% HBM peak); Huffman enc/dec GB/s; comp ratio",
        "value": round(value, 3), "unit": "GB/s (compressed-cache bytes consumed per second by one decode-attention pass)",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8 symbols, fp16 dequantized values, fp32 accumulate",
        "data": "synthetic", "config": {"workload": "%s: %s" % (args.workload, cfg["desc"]),
                                        "k_quant": "per-channel, 64-token blocks", "v_quant": "per-token",
                                        "compressed_bytes": {"k": kb, "v": vb}, "fp16_bytes_per_tensor": 2 * numel,
                                        "compression_ratio": {"k": round(kctx.get_cr(), 3), "v": round(vctx.get_cr(), 3)},
                                        "fp16_equivalent_GBs": round(4 * numel / (ms_per_step * 1e-3) / 1e9, 1),
                                        "pct_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
                                        "event_ms_per_step": res["event_ms"], "cache_copies_cycled": n_copies,
                                        "untimed_settle_seconds": args.settle_seconds,
                                        "kernels_ms": {"fused_k": round(k_ms, 4), "fused_v": round(v_ms, 4)},
                                        "arithmetic": "every (sym + min) * scale rounded to fp16 as the reference's dequantizer rounds it "
                                                      "(models/cache/kvcomp_encode.py:146), fp32 accumulation: within 1e-3 of fp32 attention over "
                                                      "that fp16 cache (checked in this run before timing); unrounded_mode keeps the products in fp32",
                                        "check_max_error": err,
                                        "graph_replay_ms_per_step": None if graph_ms is None else round(graph_ms, 4),
                                        "unrounded_mode": unrounded, "eb_k_sweep": sweep,
                                        "symbols_per_s": {"fused_k": round(numel / k_ms * 1e3), "fused_v": round(numel / v_ms * 1e3)},
                                        "first_store_ms": round(t_store * 1e3, 2), "codec": rates},
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": measured_traffic(args.workload, dom)},
    }
    if args.workload == DEFAULT_WORKLOAD and args.eb_k is None and not args.no_other_configs:
        attns = at = res = None                        # the copies of this cache are released first
        torch.cuda.empty_cache()
        static = KVCompCacheConfigStatic.config
        result["config"]["other_configs"] = other_configs(args)
        KVCompCacheConfigStatic.config = static
    if not args.no_cpu_baseline:
        log("[bench] timing the CPU restatement of the reference's path ...")
        k_head = make_kv(dict(cfg, T=min(T, 2048)), torch.device("cpu"))[0]
        result["cpu_baseline"] = cpu_baseline(kctx, q, k_head, cfg)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
