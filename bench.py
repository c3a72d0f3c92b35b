#!/usr/bin/env python3
"""Benchmark of the PackKV hot path on one MI355X.

A step = one fused decompress-attention decode (one layer, one query token per sequence) over a
compressed KV cache resident in HBM.  Workload (BASELINE.json configs[1]): batch 16, 32 query /
8 KV heads, head_dim 128, 32768 cached tokens per sequence, fp16, K ~ N(0,1) with four outlier
channels x10, V ~ N(0,1), per-token quantisation at relative step 0.1, 64-token quant blocks.

Prints ONE JSON line: the headline metric (us per layer, lower is better) with `roofline`
(HBM, algorithmic compressed bytes / measured kernel time) and `cpu_baseline` (the
decompress-then-attend path restated in PyTorch CPU ops, timed on this host on a bounded
sample), plus encode / unpack throughput measured in the same run.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0   # MI355X HBM3E, published peak

# HBM bytes per launch of the decode kernel on the default workload, from two rocprofv3 --pmc runs
# (FETCH_SIZE 208456 and WRITE_SIZE 2542 KiB per dispatch), each scaled by what the same counter read
# for a plain 256 MiB device copy in the same run (131093 -> factor 1.99969; 262144 -> factor 1.0);
# the summary with the commands is profiles/attn_dma_kernel_config1.md.  It is a recorded
# measurement, not something this script can observe, so it is reported for that workload only.
DEFAULT_TRAFFIC_BYTES = int((208456 * (262144 / 131093) + 2542 * 1.0) * 1024)
TRAFFIC_SOURCE = ("recorded rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE measurement of this workload "
                  "(profiles/attn_dma_kernel_config1.md), not observed by this run")


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--preheat-ms", type=float, default=300.0,
                    help="run the step untimed for this long before the warmup steps, so that the GPU's power "
                         "management has reached its sustained state (the first ~10 ms after a quiet period run at "
                         "lower clocks: 50 steps measured cold give 172 us/layer, 1000 steps 146 us); 0 switches it off")
    ap.add_argument("--batch", type=int, default=16)
    ap.add_argument("--ctx", type=int, default=32768)
    ap.add_argument("--hq", type=int, default=32)
    ap.add_argument("--hkv", type=int, default=8)
    ap.add_argument("--rel", type=float, default=0.1)
    ap.add_argument("--window", type=int, default=0, help="uncompressed fp16 tail tokens")
    ap.add_argument("--variant", type=int, default=0)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="skip encode / unpack timing")
    ap.add_argument("--no-sanity", action="store_true",
                    help="do not stop when the kernel disagrees with the plain kernel (development builds that switch "
                         "parts of the kernel off, -DPKV_ATTN_PROBE: their results are wrong by design)")
    ap.add_argument("--no-config-legs", action="store_true",
                    help="skip the configs[4] loop and the configs[3] decoder legs of the default run")
    ap.add_argument("--layers", type=int, default=0,
                    help="instead of the single-layer step: a decode loop over this many layers through the growing "
                         "compressed cache (configs[4] is --layers 32 --batch 4 --ctx 131072); prints its own JSON line")
    ap.add_argument("--e2e", action="store_true",
                    help="instead of the single-layer step: greedy decoding on a random-init decoder of Qwen3-8B shape "
                         "through the compressed cache (configs[3]: --e2e --batch 32 --ctx 8192 --steps 256); --e2e-layers "
                         "and --e2e-dense-steps scale it; prints its own JSON line")
    ap.add_argument("--sweep", action="store_true",
                    help="instead of the single-layer step: the repack + bit-pack sweep of configs[2] (--sweep --hkv 8 "
                         "--ctx 16384): compression ratios over pack sizes 16..256, code widths 2..8 bits and the three "
                         "repacking methods, and the block codec's encode / decode rates per width; prints its own JSON line")
    ap.add_argument("--e2e-layers", type=int, default=36)
    ap.add_argument("--e2e-dense-steps", type=int, default=4,
                    help="steps of the decompress-then-attend path timed beside the fused one (on a copy of the run)")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run one plain 256 MiB device copy (a kernel of known traffic to scale "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings by)")
    return ap.parse_args()


def event_time_ms(torch, fn, iters):
    fn()                                   # one untimed call: first-use effects stay out of the figure
    s = torch.cuda.Event(enable_timing=True)
    e = torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(iters):
        fn()
    e.record()
    e.synchronize()
    return s.elapsed_time(e) / iters


def cpu_baseline(torch, args, k1, v1, q1, threads=None, passes=5, warm=2):
    """Decompress-then-attend for a sample of the sequences in PyTorch CPU ops (the checker's restatement of
    utils/compute.py:173-179 + models/llama.py:189-212), median of `passes` after `warm` warm-ups, scaled to the
    batch: about ten seconds of host work at the default workload.  threads: torch's thread count for the
    measurement (None = all the cores torch uses by default)."""
    from oracle import quant as oq
    all_threads = torch.get_num_threads()
    if threads:
        torch.set_num_threads(threads)
    ck, zk, sk = oq.quant_ints(k1, 64, args.rel)
    cv, zv, sv = oq.quant_ints(v1, 64, args.rel)
    qq = q1.unsqueeze(2)

    def step():
        kd, vd = oq.dequant(ck, zk, sk), oq.dequant(cv, zv, sv)
        return oq.eager_attention(qq, kd, vd)

    for _ in range(warm):
        step()
    ts = []
    for _ in range(passes):
        t0 = time.perf_counter()
        step()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    n = k1.shape[0]
    per_seq = ts[len(ts) // 2] / n
    used = torch.get_num_threads()
    torch.set_num_threads(all_threads)
    return {
        "value": per_seq * args.batch * 1e6, "unit": "us/layer", "cores": used,
        "kind": "port",
        "sample": "%d of %d sequences (dequantise + eager attention, %d tokens each), median of %d passes, scaled x%g"
                  % (n, args.batch, k1.shape[2], passes, args.batch / n),
    }


def cpu_encoder(torch, args, k1):
    """Single-thread scalar encoder on the host: the reference's own k_encode_cpu when its build is
    present (oracle/_ref), else the restated C codec."""
    import numpy as np
    from oracle import codec, quant as oq
    T = min(k1.shape[2], 4096)
    c, _, _ = oq.quant_ints(k1[:, :, :T], 64, args.rel)
    cm = oq.code_matrix(c).numpy()
    kind = "reference" if codec.have_ref() else "port"
    enc = codec.ref() if codec.have_ref() else codec.oracle()
    try:
        enc.encode(1, cm, 64, 128, 4)
    except RuntimeError:
        kind, enc = "port", codec.oracle()
    t0 = time.perf_counter()
    _, _, size = enc.encode(1, cm, 64, 128, 4)
    dt = time.perf_counter() - t0
    return {"value": cm.size * 2 / dt / 1e9, "unit": "GB/s of fp16 input", "cores": 1, "kind": kind,
            "sample": "K codes of 1 sequence x %d tokens (%d channels), bit-pack only" % (T, cm.shape[1])}


def decode_loop(torch, args, dev):
    """Every layer's cache is prefilled with --ctx tokens through PackKVCompressedCache.update (residual window
    policy of the reference: all but 128..191 tokens are compressed), then a decode step = for every layer: append
    one token, attend.  Reports us per token over all layers, the share of HBM peak on the algorithmic bytes, the
    bytes the caches hold and the peak device memory."""
    from packkv_amd import synth
    from packkv_amd.cache import PackKVCacheConfig, PackKVCompressedCache
    B, Hq, Hkv, T, L = args.batch, args.hq, args.hkv, args.ctx, args.layers
    cfg = PackKVCacheConfig(64, 192, args.rel, args.rel)
    cache = PackKVCompressedCache(B, Hkv, 128, L, cfg, max_tokens=T + 1024, device=dev)
    torch.cuda.reset_peak_memory_stats()
    for layer in range(L):
        k, v = synth.make_kv(B, Hkv, T, seed=layer, device=dev)
        cache.update(k, v, layer, return_dense=False)
        del k, v
    torch.cuda.synchronize()
    q = synth.make_q(B, Hq, seed=1, device=dev)
    kn, vn = synth.make_kv(B, Hkv, 1, seed=7, device=dev)
    outs = [torch.empty_like(q) for _ in range(L)]

    def token():
        for layer in range(L):
            cache.update(kn, vn, layer, return_dense=False)
            cache.attend(q, layer, out=outs[layer])

    def algo_bytes():
        n = 0
        for lay in cache.layers:
            for side in (lay.k, lay.v):
                n += side.used + side.tokens // 128 * side.blocks_per_tile * 8 + 4 * B * side.tokens
            n += 2 * 2 * B * Hkv * lay.win_len * 128 + 2 * 2 * B * Hq * 128
        return n

    for _ in range(args.warmup):
        token()
    torch.cuda.synchronize()
    bytes_step = algo_bytes()
    comp0, win0, seq0 = cache.layers[0].k.tokens, cache.layers[0].win_len, cache.get_seq_length(0)   # at the start of timing
    t0 = time.perf_counter()
    for _ in range(args.steps):
        token()
    torch.cuda.synchronize()
    us_token = (time.perf_counter() - t0) * 1e6 / args.steps
    lay0 = cache.layers[0]
    result = {
        "metric": "compressed-cache decode us/token over all layers", "value": us_token, "unit": "us/token",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": us_token / 1e3,
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "%d layers, batch %d, %d q / %d KV heads, head_dim 128, %d cached tokens per sequence "
                               "(%d compressed + %d in the 16-bit window at the start of timing), rel %.3g; a step appends "
                               "one token to every layer and attends" % (L, B, Hq, Hkv, seq0, comp0, win0, args.rel)},
        "tokens_per_s": B / (us_token * 1e-6),
        "roofline": {"bound": "hbm", "achieved": bytes_step / (us_token * 1e-6) / 1e9, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": bytes_step / (us_token * 1e-6) / 1e9 / HBM_PEAK_GBS, "traffic": None,
                     "algorithmic_bytes": bytes_step},
        "kv_bytes": cache.cache_bytes(), "fp16_kv_bytes": L * 2 * B * Hkv * cache.get_seq_length(0) * 128 * 2,
        "peak_device_bytes": torch.cuda.max_memory_allocated(),
        "cpu_baseline": None,
    }
    return result


def e2e_decode(torch, args, dev):
    """configs[3]: a random-init decoder of Qwen3-8B shape (bf16 weights ~ N(0, 0.02)), a random-token prompt of
    --ctx tokens per sequence, --steps greedy tokens; the cache compresses a 64-token cut whenever its 16-bit buffer
    reaches 192 tokens.  Reports decode tokens/s of the fused path, the prompt pass, the bytes the caches hold, and
    a few steps of the reference's decompress-then-attend on the same cache for scale."""
    from packkv_amd.cache import PackKVCacheConfig
    from packkv_amd.decoder import DecoderShape, ShapedDecoder
    B, T, steps = args.batch, args.ctx, args.steps
    shape = DecoderShape(layers=args.e2e_layers, q_heads=args.hq, kv_heads=args.hkv)
    t0 = time.perf_counter()
    model = ShapedDecoder(shape, dtype=torch.bfloat16, device=dev, seed=0)
    torch.cuda.synchronize()
    build_s = time.perf_counter() - t0
    ids = torch.randint(0, shape.vocab, (B, T), generator=torch.Generator().manual_seed(1)).to(dev)
    cache = model.new_cache(B, T + steps + args.e2e_dense_steps + 256, PackKVCacheConfig(64, 192, args.rel, args.rel))
    torch.cuda.reset_peak_memory_stats()
    t0 = time.perf_counter()
    logits = model.prefill(ids, cache)
    torch.cuda.synchronize()
    prefill_s = time.perf_counter() - t0
    for _ in range(args.warmup):               # untimed steps (they stay in the cache; the timed ones follow)
        logits = model.forward(logits.argmax(dim=-1, keepdim=True), cache, attention="fused")
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        logits = model.forward(logits.argmax(dim=-1, keepdim=True), cache, attention="fused")
    torch.cuda.synchronize()
    step_ms = (time.perf_counter() - t0) * 1e3 / steps
    kv_bytes, seq = cache.cache_bytes(), cache.get_seq_length(0)
    lay0 = cache.layers[0]
    dense_ms = None
    if args.e2e_dense_steps > 0:
        nxt = logits.argmax(dim=-1, keepdim=True)
        model.forward(nxt, cache, attention="dense")
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.e2e_dense_steps):
            model.forward(nxt, cache, attention="dense")
        torch.cuda.synchronize()
        dense_ms = (time.perf_counter() - t0) * 1e3 / args.e2e_dense_steps
    result = {
        "metric": "end-to-end greedy decode tokens/s with the compressed cache", "value": B / (step_ms * 1e-3),
        "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup, "ms_per_step": step_ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "random-init decoder, %d layers, hidden %d, %d q / %d KV heads, head_dim 128, vocabulary %d; "
                               "batch %d, %d-token random prompt, %d greedy tokens (+%d untimed), rel %.3g, 64-token cuts, "
                               "16-bit buffer 128..191 tokens" % (shape.layers, shape.hidden, shape.q_heads, shape.kv_heads,
                                                                  shape.vocab, B, T, steps, args.warmup, args.rel)},
        "prefill_s": prefill_s, "prefill_tokens_per_s": B * T / prefill_s, "model_build_s": build_s,
        "cached_tokens": seq, "compressed_tokens": lay0.k.tokens,
        "kv_bytes": kv_bytes, "fp16_kv_bytes": shape.layers * 2 * B * shape.kv_heads * seq * 128 * 2,
        "decompress_then_attend_ms_per_step": dense_ms,
        "peak_device_bytes": torch.cuda.max_memory_allocated(),
        "roofline": None, "cpu_baseline": None,
    }
    return result


SWEEP_RELS = (0.5, 0.2, 0.1, 0.05, 0.025, 0.0125, 0.00625)      # code widths 2, 3, 4, 5, 6, 7, 8 bits
SWEEP_PACKS = (16, 32, 64, 128, 256)


def pack_sweep(torch, H, T, dev, rels=SWEEP_RELS, packs=SWEEP_PACKS, time_codec=True, kv=None):
    """configs[2]: one layer of H KV heads x 128 x T tokens, K with a per-channel scale drawn log-uniform in
    [0.1, 10], V ~ N(0, 1).  For every error bound (one per code width) the tensors are quantised once; every
    (pack size, repacking method) is then priced with the reference's size model (`repack_and_encode`,
    utils/compute.py:329-357: integers, so the ratios are the reference's wherever its token order is defined),
    and the real block codec is run and timed on the same codes at every pack length."""
    from packkv_amd import ops, synth
    hid = H * 128
    k, v = kv if kv is not None else synth.make_kv(1, H, T, seed=2, device=dev, k_mode="channel_scale")
    fp16 = T * hid * 2
    rows, codec = [], []
    for rel in rels:
        bits = ops.bits_for_rel(rel)
        mats = []
        for x in (k, v):
            scale, zero = ops.quant_params(x, rel)
            mats.append(ops.quantize(x, scale, zero)[0])
        kc, vc = mats
        for pack in packs:
            for method in ("none", "median", "greedy"):
                bs = max(64, pack)
                if method == "greedy" and bs > 256:
                    continue
                k_pre, v_pre, k_aft, v_aft = ops.repack_and_encode(kc, vc, pack, method, bs)
                rows.append({"rel": rel, "bits": bits, "pack": pack, "method": method, "block": bs,
                             "k_bytes": k_aft, "v_bytes": v_aft, "k_cr": fp16 / k_aft, "v_cr": fp16 / v_aft})
        if time_codec:
            # the real block codec at every pack length (16 = the reference's format; longer packs = this build's
            # extension of it): stream bytes - 8 per block equal the size model's bytes of the "none" rows above
            back = torch.empty_like(kc)
            gbs = lambda ms: T * hid / (ms * 1e-3) / 1e9
            for pack in packs:
                if T % (8 * pack):
                    continue
                row = {"rel": rel, "bits": bits, "pack": pack}
                for name, is_k, mat in (("k", True, kc), ("v", False, vc)):
                    ctx_blk, hid_blk = ops.long_block_shape(is_k, pack)
                    nblk = (T // ctx_blk) * (hid // hid_blk)
                    stream = torch.empty(nblk * ops.block_bound_p(pack, bits), dtype=torch.uint8, device=dev)
                    info = torch.empty(nblk, 2, dtype=torch.uint32, device=dev)
                    size = ops.encode_p(is_k, mat, stream, info, pack, bits)
                    enc = event_time_ms(torch, lambda: ops.encode_p(is_k, mat, stream, info, pack, bits, want_size=False), 10)
                    dec = event_time_ms(torch, lambda: ops.decode_p(is_k, stream, info, back, pack, bits), 10)
                    assert torch.equal(back, mat)
                    model = [r for r in rows if r["rel"] == rel and r["pack"] == pack and r["method"] == "none"][0]
                    assert size - 8 * nblk == model[name + "_bytes"], (rel, pack, name)
                    row.update({name + "_stream_bytes": size, name + "_cr": fp16 / size,
                                name + "_encode_gbs_codes": gbs(enc), name + "_decode_gbs_codes": gbs(dec)})
                codec.append(row)
    return {"metric": "repack + bit-pack sweep", "n_gpus": 1, "data": "synthetic", "dtype": "u8",
            "config": {"workload": "configs[2]: %d KV heads x 128 x %d tokens, K per-channel scale log-uniform in "
                                   "[0.1, 10], V ~ N(0, 1); sizes by the reference's size model (payload + pack "
                                   "metadata, no quantiser parameters), ratios against fp16" % (H, T)},
            "rows": rows, "codec": codec}


def gemv_surface(torch, ops, synth, dev):
    """The reference's own GPU ops at the shape its throughput script runs (one sequence of Llama-3.1-8B shape:
    8 KV heads, 65536 cached tokens, K at rel 0.1 = 4-bit codes, V at rel 0.2 = 3-bit codes) and by its definition:
    fp16 bytes of the uncompressed tensor / kernel time, K = kq_mat_vec_mul + fused_kq, V = wv_mat_vec_mul +
    fused_wv, every op timed by the events inside its launcher (scripts/figure/throughput.py:124-138), beside
    torch.matmul on the fp16 tensor."""
    H, T = 8, 65536
    hid = H * 128
    k, v = synth.make_kv(1, H, T, seed=5, device=dev)
    ke, ve = ops.k_quant_encode(k, 0.1, 4), ops.v_quant_encode(v, 0.2, 3)
    q = torch.randn(H, 128, device=dev).half()
    t = torch.zeros(H, T, dtype=torch.float16, device=dev)
    w = torch.softmax(torch.randn(H, T, device=dev), dim=1).half()
    term = torch.zeros(H, 128, dtype=torch.float32, device=dev)
    our_kq, our_wv = torch.empty_like(t), torch.empty(H, 128, dtype=torch.float16, device=dev)
    kz, ks = ke["zero"].reshape(-1), ke["scale"].reshape(-1)
    vz, vs = ve["zero"].reshape(-1), ve["scale"].reshape(-1)
    term16 = term.half()

    def med(fn):
        xs = sorted(fn() for _ in range(31))
        return xs[15]

    kq = med(lambda: ops.kq_mat_vec_mul(ke["stream"], ke["info"], q, t, T, hid, 64, 128, 4))
    fkq = med(lambda: ops.fused_kq(our_kq, q, kz, ks, t))
    wv = med(lambda: ops.wv_mat_vec_mul(ve["stream"], ve["info"], w, term, T, hid, 128, 64, 3))
    fwv = med(lambda: ops.fused_wv(our_wv, w, vz, vs, term16))
    k3, v3 = k[0], v[0]                                   # [H, T, 128]
    mk = event_time_ms(torch, lambda: torch.matmul(k3, q.unsqueeze(2)), 30)
    mv = event_time_ms(torch, lambda: torch.matmul(w.unsqueeze(1), v3), 30)
    fp16 = T * hid * 2
    gib = lambda ms: fp16 / 2 ** 30 / (ms * 1e-3)
    return {"shape": "1 sequence, 8 KV heads x 128, 65536 tokens; K 4-bit (rel 0.1), V 3-bit (rel 0.2)",
            "kq_ms": kq, "fused_kq_ms": fkq, "wv_ms": wv, "fused_wv_ms": fwv,
            "k_gibs_of_fp16": gib(kq + fkq), "v_gibs_of_fp16": gib(wv + fwv),
            "torch_matmul_k_ms": mk, "torch_matmul_v_ms": mv,
            "torch_matmul_k_gibs": gib(mk), "torch_matmul_v_gibs": gib(mv)}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (--gpus %d refused)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    import torch
    from packkv_amd import ops, synth

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.layers > 0:
        print(json.dumps(decode_loop(torch, args, dev)))
        return
    if args.e2e:
        print(json.dumps(e2e_decode(torch, args, dev)))
        return
    if args.sweep:
        print(json.dumps(pack_sweep(torch, args.hkv, args.ctx, dev)))
        return
    B, Hq, Hkv, T, Tw = args.batch, args.hq, args.hkv, args.ctx, args.window
    Tc = T - Tw
    assert Tc % 128 == 0, "compressed tokens must be a multiple of 128"

    k, v = synth.make_kv(B, Hkv, T, seed=0, device=dev)
    q = synth.make_q(B, Hq, seed=1, device=dev)
    kc, vc = (k[:, :, :Tc].contiguous(), v[:, :, :Tc].contiguous()) if Tw else (k, v)
    kw = k[:, :, Tc:].contiguous() if Tw else None
    vw = v[:, :, Tc:].contiguous() if Tw else None

    bits = ops.bits_for_rel(args.rel)
    ke = ops.k_quant_encode(kc, args.rel, bits)
    ve = ops.v_quant_encode(vc, args.rel, bits)
    hidden = B * Hkv * 128
    nblk_k, nblk_v = (Tc // 64) * (hidden // 128), (Tc // 128) * (hidden // 64)
    fp16_bytes = 2 * Tc * hidden * 2
    algo_bytes = (ke["size"] + ve["size"] + 8 * (nblk_k + nblk_v) + 8 * B * Tc
                  + 2 * 2 * B * Hkv * Tw * 128 + 2 * 2 * B * Hq * 128)

    out = torch.empty_like(q)

    if args.calib_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)           # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    def step():
        ops.attn_decode(q, ke, ve, kw, vw, out=out, variant=args.variant)

    # Before anything is timed: the kernel under test against the library's plain kernel (variant 1: unpack to a code
    # tile, fp32 arithmetic) on the whole batch -- both evaluate the same exact formula, so they may differ by the
    # fast kernel's fp16 weights and one output rounding only.  A broken kernel is not timed.
    step()
    plain = ops.attn_decode(q, ke, ve, kw, vw, variant=1)
    diff = (out.float() - plain.float()).abs()
    bound = 1e-3 + 2.0 ** -9 * plain.float().abs()
    sanity = {"max_abs_diff_vs_plain_kernel": float(diff.max()), "ok": bool((diff <= bound).all())}
    if not args.no_sanity and (not sanity["ok"] or not bool(torch.isfinite(out.float()).all())):
        raise SystemExit("bench: the attention kernel disagrees with the plain kernel: %r" % (sanity,))
    del plain, diff, bound

    preheat_steps = 0
    t_end = time.perf_counter() + args.preheat_ms * 1e-3
    while time.perf_counter() < t_end:
        for _ in range(20):
            step()
        torch.cuda.synchronize()
        preheat_steps += 20
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    s_ev = torch.cuda.Event(enable_timing=True)
    e_ev = torch.cuda.Event(enable_timing=True)
    s_ev.record()
    for _ in range(args.steps):
        step()
    e_ev.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_step = wall * 1e3 / args.steps
    ms_kernel = s_ev.elapsed_time(e_ev) / args.steps

    default_workload = (B, Hq, Hkv, T, Tw, args.variant) == (16, 32, 8, 32768, 0, 0) and abs(args.rel - 0.1) < 1e-9
    result = {
        "metric": "fused decompress-attn decode us/layer",
        "value": ms_step * 1e3, "unit": "us/layer", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_step, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic", "preheat": {"ms": args.preheat_ms, "steps": preheat_steps},
        "config": {"workload": "configs[1]: GQA decode, batch %d, %d q / %d KV heads, head_dim 128, %d tokens"
                               " (%d compressed + %d fp16 tail), rel %.3g, %d-bit codes"
                               % (B, Hq, Hkv, T, Tc, Tw, args.rel, bits),
                   "variant": args.variant},
        "tokens_per_s": B / (ms_step * 1e-3),
        "roofline": {"bound": "hbm", "achieved": algo_bytes / (ms_kernel * 1e-3) / 1e9, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": algo_bytes / (ms_kernel * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "traffic": DEFAULT_TRAFFIC_BYTES if default_workload else None,
                     "traffic_source": TRAFFIC_SOURCE if default_workload else None,
                     "kernel_ms": ms_kernel, "algorithmic_bytes": algo_bytes},
        "sanity": sanity,
        "compression": {"k_bytes": ke["size"], "v_bytes": ve["size"], "fp16_bytes": fp16_bytes,
                        "ratio_k": fp16_bytes / 2 / ke["size"], "ratio_v": fp16_bytes / 2 / ve["size"]},
    }

    if not args.no_extras:
        # encode: fused quantize + bit-pack, fp16 in -> stream out (GB/s of fp16 input consumed)
        x_bytes = Tc * hidden * 2
        k_ms = event_time_ms(torch, lambda: ops.k_quant_encode(kc, args.rel, bits, ke["stream"], ke["info"],
                                                               want_size=False), 20)
        v_ms = event_time_ms(torch, lambda: ops.v_quant_encode(vc, args.rel, bits, ve["stream"], ve["info"],
                                                               want_size=False), 20)
        codes = torch.empty(Tc, hidden, dtype=torch.uint8, device=dev)
        uk_ms = event_time_ms(torch, lambda: ops.k_decode(ke["stream"], ke["info"], codes, 64, 128, bits), 5)
        uv_ms = event_time_ms(torch, lambda: ops.v_decode(ve["stream"], ve["info"], codes, 128, 64, bits), 5)
        # token repacking + analytic size on the code matrices (K codes in `codes`, V codes beside them)
        codes_v = torch.empty(Tc, hidden, dtype=torch.uint8, device=dev)
        ops.k_decode(ke["stream"], ke["info"], codes, 64, 128, bits)
        ops.v_decode(ve["stream"], ve["info"], codes_v, 128, 64, bits)
        # the block codec alone, code matrix -> stream (the reference's k_encode_cpu / v_encode_cpu on the device)
        ck_ms = event_time_ms(torch, lambda: ops.k_encode(codes, ke["stream"], ke["info"], 64, 128, bits, want_size=False), 3)
        cv_ms = event_time_ms(torch, lambda: ops.v_encode(codes_v, ve["stream"], ve["info"], 128, 64, bits, want_size=False), 3)
        rp_ms = event_time_ms(torch, lambda: ops.median_repacking(codes, codes_v, 64), 3)
        bp_ms = event_time_ms(torch, lambda: ops.bit_pack_bytes(codes, 16), 3)
        g_rows = min(Tc, 8192)      # 128 blocks of 64 tokens x 2 x 16384 channels: the shape the kernel's figures are quoted on
        gr_ms = event_time_ms(torch, lambda: ops.greedy_repacking(codes[:g_rows], codes_v[:g_rows], 16, 64), 2)
        result["repack"] = {
            "greedy_repack_ms": gr_ms, "greedy_repack_rows": g_rows,
            "median_repack_ms": rp_ms, "median_repack_gbs": 5 * Tc * hidden / (rp_ms * 1e-3) / 1e9,   # V read twice, K once, both written
            "bit_pack_size_ms": bp_ms, "bit_pack_size_gbs": Tc * hidden / (bp_ms * 1e-3) / 1e9,
        }
        # packs longer than 16 tokens (this build's extension of the format) on the same 2 x 512 MiB of codes: the real
        # codec at every pack length, beside the 16-token codec's figures above (K decode 1.0 = as fast as that one)
        long_packs = {}
        back = torch.empty_like(codes)
        for pack in (32, 64, 128, 256):
            row = {}
            for name, is_k, mat, ref_enc, ref_dec in (("k", True, codes, ck_ms, uk_ms), ("v", False, codes_v, cv_ms, uv_ms)):
                ctx_blk, hid_blk = ops.long_block_shape(is_k, pack)
                if Tc % ctx_blk:
                    continue
                info_p = torch.empty((Tc // ctx_blk) * (hidden // hid_blk), 2, dtype=torch.uint32, device=dev)
                stream_p = ke["stream"] if is_k else ve["stream"]
                if stream_p.numel() < info_p.shape[0] * ops.block_bound_p(pack, bits):
                    stream_p = torch.empty(info_p.shape[0] * ops.block_bound_p(pack, bits), dtype=torch.uint8, device=dev)
                size_p = ops.encode_p(is_k, mat, stream_p, info_p, pack, bits)
                e_ms = event_time_ms(torch, lambda: ops.encode_p(is_k, mat, stream_p, info_p, pack, bits, want_size=False), 3)
                d_ms = event_time_ms(torch, lambda: ops.decode_p(is_k, stream_p, info_p, back, pack, bits), 3)
                row.update({name + "_encode_ms": e_ms, name + "_decode_ms": d_ms, name + "_stream_bytes": size_p,
                            name + "_encode_vs_16": ref_enc / e_ms, name + "_decode_vs_16": ref_dec / d_ms})
                del info_p
            long_packs["pack %d" % pack] = row
        # (the long-pack encodes overwrote the streams: put the 16-token streams back for what follows)
        ops.k_quant_encode(kc, args.rel, bits, ke["stream"], ke["info"], want_size=False)
        ops.v_quant_encode(vc, args.rel, bits, ve["stream"], ve["info"], want_size=False)
        result["long_packs"] = long_packs
        del codes, codes_v, back
        # median repacking inside the encode: the order from V itself (V's parameters kept), then the fused encoders
        # on the permuted rows -- against the plain fused encode above, all on preallocated buffers
        if Hkv <= 8 and bits <= 6:
            perm, vs_nat, vz_nat = ops.median_order(vc, args.rel, bits, 64, want_params=True)
            # five legs timed the same way, one after the other (3 untimed + 20 timed calls each), so that the ratio
            # compares like with like: the plain encoders again, then order, K and V on the permuted rows
            def leg(fn):
                for _ in range(2):
                    fn()
                return event_time_ms(torch, fn, 20)
            k2_ms = leg(lambda: ops.k_quant_encode(kc, args.rel, bits, ke["stream"], ke["info"], want_size=False))
            v2_ms = leg(lambda: ops.v_quant_encode(vc, args.rel, bits, ve["stream"], ve["info"], want_size=False))
            mo_ms = leg(lambda: ops.median_order(vc, args.rel, bits, 64, want_params=True))
            kp_ms = leg(lambda: ops._quant_encode(True, kc, args.rel, bits, ke["stream"], ke["info"], False,
                                                  False, perm, 64))
            vp_ms = leg(lambda: ops._quant_encode(False, vc, args.rel, bits, ve["stream"], ve["info"], False,
                                                  False, perm, 64, (vs_nat, vz_nat)))
            # (the timed calls overwrote the streams with the repacked ones: restore the natural order for what follows)
            ops.k_quant_encode(kc, args.rel, bits, ke["stream"], ke["info"], want_size=False)
            ops.v_quant_encode(vc, args.rel, bits, ve["stream"], ve["info"], want_size=False)
            result["repack"].update({
                "fused_median_order_ms": mo_ms, "fused_k_encode_ms": kp_ms, "fused_v_encode_ms": vp_ms,
                "fused_median_encode_ms": mo_ms + kp_ms + vp_ms,
                "plain_k_encode_ms": k2_ms, "plain_v_encode_ms": v2_ms,
                "fused_median_encode_vs_plain": (mo_ms + kp_ms + vp_ms) / (k2_ms + v2_ms)})
            del perm, vs_nat, vz_nat
        enc_algo_k = x_bytes + ke["size"] + 8 * nblk_k + 4 * B * Tc
        enc_algo_v = x_bytes + ve["size"] + 8 * nblk_v + 4 * B * Tc
        result["encode"] = {
            "k_ms": k_ms, "v_ms": v_ms,
            "k_gbs_fp16_in": x_bytes / (k_ms * 1e-3) / 1e9, "v_gbs_fp16_in": x_bytes / (v_ms * 1e-3) / 1e9,
            "k_roofline_frac": enc_algo_k / (k_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "v_roofline_frac": enc_algo_v / (v_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
        }
        result["codec_encode"] = {"k_ms": ck_ms, "v_ms": cv_ms, "k_gbs_codes": Tc * hidden / (ck_ms * 1e-3) / 1e9,
                                  "v_gbs_codes": Tc * hidden / (cv_ms * 1e-3) / 1e9}
        result["unpack"] = {
            "k_ms": uk_ms, "v_ms": uv_ms,
            "k_gbs": (ke["size"] + 8 * nblk_k + Tc * hidden) / (uk_ms * 1e-3) / 1e9,
            "v_gbs": (ve["size"] + 8 * nblk_v + Tc * hidden) / (uv_ms * 1e-3) / 1e9,
        }
        # what this GPU sustains on plain traffic, beside the published 8 TB/s the roofline is priced against:
        # a 1 GiB device-to-device copy (read + write) and the read-only parameter pass over the same 1 GiB
        src = kc.view(torch.uint8).reshape(-1)
        dst = torch.empty_like(src)
        cp_ms = event_time_ms(torch, lambda: dst.copy_(src), 5)
        rd_ms = event_time_ms(torch, lambda: ops.quant_params(kc, args.rel), 5)
        result["hbm_probe"] = {"copy_gbs": 2 * src.numel() / (cp_ms * 1e-3) / 1e9,
                               "read_gbs": src.numel() / (rd_ms * 1e-3) / 1e9, "bytes": src.numel()}
        del dst

    if not args.no_extras and default_workload:
        # configs[1] names three error bounds; the line above is the middle one.  The other two on the same tensors:
        # fused encode, unpack and the decode step (5-bit codes at 0.05 are this build's extension of the format)
        other = {}
        for rel2 in (0.05, 0.2):
            b2 = ops.bits_for_rel(rel2)
            ke2, ve2 = ops.k_quant_encode(kc, rel2, b2), ops.v_quant_encode(vc, rel2, b2)
            out2 = torch.empty_like(q)
            f2 = lambda: ops.attn_decode(q, ke2, ve2, out=out2)
            for _ in range(100):
                f2()
            a_ms = event_time_ms(torch, f2, 300)
            k2 = event_time_ms(torch, lambda: ops.k_quant_encode(kc, rel2, b2, ke2["stream"], ke2["info"], want_size=False), 5)
            v2 = event_time_ms(torch, lambda: ops.v_quant_encode(vc, rel2, b2, ve2["stream"], ve2["info"], want_size=False), 5)
            codes2 = torch.empty(Tc, hidden, dtype=torch.uint8, device=dev)
            uk2 = event_time_ms(torch, lambda: ops.k_decode(ke2["stream"], ke2["info"], codes2, 64, 128, b2), 5)
            uv2 = event_time_ms(torch, lambda: ops.v_decode(ve2["stream"], ve2["info"], codes2, 128, 64, b2), 5)
            bytes2 = ke2["size"] + ve2["size"] + 8 * (nblk_k + nblk_v) + 8 * B * Tc + 2 * 2 * B * Hq * 128
            other["rel %.3g" % rel2] = {
                "bits": b2, "attn_us": a_ms * 1e3, "attn_roofline_frac": bytes2 / (a_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                "encode_k_ms": k2, "encode_v_ms": v2, "unpack_k_ms": uk2, "unpack_v_ms": uv2,
                "ratio_k": fp16_bytes / 2 / ke2["size"], "ratio_v": fp16_bytes / 2 / ve2["size"]}
            del ke2, ve2, codes2
        result["other_error_bounds"] = other
        # the same bytes as fewer, longer sequences (one layer of configs[4] is 4 x 131072 tokens): the tensors read as
        # [B / f, Hkv, f * Tc, 128], encoded and attended at that shape -- more members share a KV head there
        longer = {}
        for f in (4, 16):
            if B % f or f * Tc % 128:
                continue
            k4, v4 = kc.view(B // f, Hkv, f * Tc, 128), vc.view(B // f, Hkv, f * Tc, 128)
            ke4, ve4 = ops.k_quant_encode(k4, args.rel, bits), ops.v_quant_encode(v4, args.rel, bits)
            q4 = q[:B // f].contiguous()
            out4 = torch.empty_like(q4)
            f4 = lambda: ops.attn_decode(q4, ke4, ve4, out=out4)
            for _ in range(100):
                f4()
            a_ms = event_time_ms(torch, f4, 300)
            bytes4 = ke4["size"] + ve4["size"] + 8 * (nblk_k + nblk_v) + 8 * B * Tc + 2 * 2 * (B // f) * Hq * 128
            longer["batch %d x %d tokens" % (B // f, f * Tc)] = {
                "attn_us": a_ms * 1e3, "attn_roofline_frac": bytes4 / (a_ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
            del ke4, ve4
        result["longer_sequences"] = longer

    if not args.no_extras and default_workload:
        result["gemv_surface"] = gemv_surface(torch, ops, synth, dev)

    if not args.no_cpu:
        ns = min(B, 16)
        k1, v1, q1 = kc[:ns].cpu(), vc[:ns].cpu(), q[:ns].cpu()
        result["cpu_baseline"] = cpu_baseline(torch, args, k1, v1, q1)
        # the same path on one host thread, on one sequence (a few seconds)
        result["cpu_baseline_1thread"] = cpu_baseline(torch, args, k1[:1], v1[:1], q1[:1], threads=1, passes=3, warm=1)
        result["cpu_encode"] = cpu_encoder(torch, args, k1[:1])
    else:
        result["cpu_baseline"] = None

    if not args.no_extras and not args.no_config_legs and default_workload:
        # the two configurations that run more than one layer, at their own sizes and in this same run: configs[4]'s
        # loop over 32 layers of the growing cache and configs[3]'s greedy decode through the decoder (both have flags
        # of their own for longer runs: --layers / --e2e).  A leg that fails reports its error instead of a figure.
        del k, v, kc, vc, ke, ve, q, out
        import copy
        import gc
        for name, fn, over in (
                ("configs4_loop", decode_loop, dict(layers=32, batch=4, ctx=131072, steps=70, warmup=5)),
                ("configs3_e2e", e2e_decode, dict(batch=32, ctx=8192, steps=64, warmup=4, e2e_dense_steps=2))):
            a2 = copy.copy(args)
            for key, val in over.items():
                setattr(a2, key, val)
            gc.collect()
            torch.cuda.empty_cache()
            t0 = time.perf_counter()
            try:
                r = fn(torch, a2, dev)
            except Exception as e:      # noqa: BLE001 -- the headline line must still be printed
                result[name] = {"error": "%s: %s" % (type(e).__name__, e)}
                continue
            if name == "configs4_loop":
                result[name] = {"us_per_token": r["value"], "us_per_layer": r["value"] / a2.layers,
                                "roofline_frac": r["roofline"]["frac"], "algorithmic_bytes": r["roofline"]["algorithmic_bytes"],
                                "tokens_per_s": r["tokens_per_s"], "kv_bytes": r["kv_bytes"], "fp16_kv_bytes": r["fp16_kv_bytes"],
                                "peak_device_bytes": r["peak_device_bytes"], "steps": r["steps"], "workload": r["config"]["workload"]}
            else:
                result[name] = {"tokens_per_s": r["value"], "ms_per_step": r["ms_per_step"], "kv_bytes": r["kv_bytes"],
                                "fp16_kv_bytes": r["fp16_kv_bytes"], "prefill_tokens_per_s": r["prefill_tokens_per_s"],
                                "decompress_then_attend_ms_per_step": r["decompress_then_attend_ms_per_step"],
                                "peak_device_bytes": r["peak_device_bytes"], "steps": r["steps"], "dtype": r["dtype"],
                                "workload": r["config"]["workload"]}
            result[name]["leg_seconds"] = time.perf_counter() - t0
    print(json.dumps(result))


if __name__ == "__main__":
    main()
