"""Benchmark of the hot path on one MI355X.

Primary line (BASELINE.json metric "bfp8_b matmul TFLOP/s ..."): the config-3 linear layer at
M=2048 -- bf16 activations [2048,4096] x bfp8_b weights [4096,14336], fused bias + GELU, fp32
accumulate -- one kernel launch per step, inputs resident in HBM.  The same JSON line carries
the pack / unpack / tilize bandwidth figures of config 2 and the decode-shape (M=32) linear under
"secondary", each with its own roofline object, and the CPU baseline timed on this host.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload linear2048|pack_bfp8|...]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import __graft_entry__ as entry  # noqa: E402

HBM_PEAK_GBS = 8000.0        # MI355X published HBM3E bandwidth
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X published dense bf16 MFMA peak


def _events_time(hip, stream, fn, steps):
    a, b = hip.Event(), hip.Event()
    a.record(stream)
    for _ in range(steps):
        fn()
    b.record(stream)
    b.sync()
    return a.elapsed_ms(b) / steps


def _wall_time(torch, fn, steps):
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def sample_sclk(torch, fn, seconds=1.2):
    """Shader clock reported by the driver while `fn` is launched back to back for `seconds`: (median MHz, samples).  The
    matrix kernels run against the board's power limit, so the clock they are given is part of the measurement."""
    import re
    import statistics
    import subprocess
    import threading
    vals, stop = [], [False]

    # the driver's own file first (no child process: a profiler's preloaded library initialises the GPU in every process it
    # is loaded into, rocm-smi's interpreter included); rocm-smi only where that file is missing
    import glob
    dpm = sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))
    preloaded = "rocprof" in os.environ.get("LD_PRELOAD", "")

    def poll():
        while not stop[0]:
            try:
                if dpm:
                    for line in open(dpm[0]).read().splitlines():
                        m = re.search(r"(\d+)\s*Mhz\s*\*", line)
                        if m:
                            vals.append(int(m.group(1)))
                elif not preloaded:
                    out = subprocess.run(["rocm-smi", "--showclocks", "--json"], stdout=subprocess.PIPE, stderr=subprocess.DEVNULL,
                                         text=True, timeout=5).stdout
                    card = next(iter(json.loads(out).values()))
                    for key, value in card.items():
                        m = re.search(r"(\d+)\s*Mhz", str(value))
                        if "sclk clock speed" in key and m:
                            vals.append(int(m.group(1)))
            except Exception:
                pass
            time.sleep(0.1)
    for _ in range(20):
        fn()
    torch.cuda.synchronize()
    th = threading.Thread(target=poll, daemon=True)
    th.start()
    t0, n = time.perf_counter(), 0
    while time.perf_counter() - t0 < seconds:
        for _ in range(50):
            fn()
        n += 50
        torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / n
    stop[0] = True
    th.join(timeout=6)
    vals = vals[1:] if len(vals) > 2 else vals          # the first sample may predate the load
    return (int(statistics.median(vals)) if vals else None), len(vals), ms


class Workload:
    """name, bound ('hbm'|'mfma'), algorithmic work per launch, fn() launching exactly one kernel."""

    def __init__(self, name, bound, work, unit_work, fn, desc, extra=None):
        self.name, self.bound, self.work, self.unit_work, self.fn, self.desc = name, bound, work, unit_work, fn, desc
        self.extra = extra or {}


def make_workloads(torch, hip, datagen, dev, names):
    s = hip.current_stream()
    out = {}
    R = C = 8192
    ntiles = (R // 32) * (C // 32)
    need_c2 = any(n in names for n in ("pack_bfp8", "unpack_bfp8", "pack_bfp4", "unpack_bfp4", "tilize_f32",
                                       "untilize_f32", "copy"))
    if need_c2:
        x = datagen.c2_outliers(R, C, seed=0).to(dev)
        y = torch.empty_like(x)
        for fmt, nm in ((hip.BFP8B, "bfp8"), (hip.BFP4B, "bfp4")):
            tb = hip.bfp_tile_bytes(fmt)
            p = torch.empty(ntiles * tb, dtype=torch.uint8, device=dev)
            hip.call("ttm_bfp_pack", hip.ptr(x), hip.F32, hip.ROW_MAJOR, hip.ptr(p), fmt, 1, R, C, s)
            work = R * C * 4 + ntiles * tb
            out["pack_" + nm] = Workload(
                "pack_" + nm, "hbm", work, "bytes",
                (lambda p=p, fmt=fmt: hip.call("ttm_bfp_pack", hip.ptr(x), hip.F32, hip.ROW_MAJOR, hip.ptr(p), fmt, 1, R, C, s)),
                "config 2: fp32 [8192,8192] row-major -> %s_b tiles (tilize fused)" % nm)
            out["unpack_" + nm] = Workload(
                "unpack_" + nm, "hbm", work, "bytes",
                (lambda p=p, fmt=fmt: hip.call("ttm_bfp_unpack", hip.ptr(p), fmt, hip.ptr(y), hip.F32, hip.ROW_MAJOR, 1, R, C, s)),
                "config 2: %s_b tiles -> fp32 [8192,8192] row-major (untilize fused)" % nm)
        out["tilize_f32"] = Workload("tilize_f32", "hbm", 2 * R * C * 4, "bytes",
                                     lambda: hip.call("ttm_tilize", hip.ptr(x), hip.ptr(y), 1, R, C, 4, s),
                                     "config 2: tilize fp32 [8192,8192]")
        out["untilize_f32"] = Workload("untilize_f32", "hbm", 2 * R * C * 4, "bytes",
                                       lambda: hip.call("ttm_untilize", hip.ptr(x), hip.ptr(y), 1, R, C, 4, s),
                                       "config 2: untilize fp32 [8192,8192]")
        out["copy"] = Workload("copy", "hbm", 2 * R * C * 4, "bytes",
                               lambda: hip.call("ttm_copy_kernel", hip.ptr(x), hip.ptr(y), R * C * 4, s),
                               "plain 16 B/lane copy of 256 MiB (measured HBM ceiling)")
    for M in (2048, 32):
        nm = "linear%d" % M
        if nm not in names:
            continue
        K, N = 4096, 14336
        a, w, bias = datagen.c3_linear(M)
        ad, wd, bd = a.to(dev), w.to(dev), bias.reshape(1, -1).to(dev)
        at = torch.empty(M * K, dtype=torch.bfloat16, device=dev)
        hip.call("ttm_tilize", hip.ptr(ad), hip.ptr(at), 1, M, K, 2, s)
        wt = torch.empty((K // 32) * (N // 32) * 1088, dtype=torch.uint8, device=dev)
        hip.call("ttm_bfp_pack", hip.ptr(wd), hip.F32, hip.ROW_MAJOR, hip.ptr(wt), hip.BFP8B, 1, K, N, s)
        bt = torch.zeros(32 * N, dtype=torch.bfloat16, device=dev)
        hip.call("ttm_tilize", hip.ptr(bd), hip.ptr(bt), 1, 1, N, 2, s)
        ot = torch.empty(M * N, dtype=torch.bfloat16, device=dev)
        torch.cuda.synchronize()
        del wd
        # decode streams the weights once per launch: ten copies are cycled (624 MB) so that every launch reads them from
        # HBM and not from the 256 MB last-level cache, as a layer stack of distinct weights would
        wts = [wt] + ([wt.clone() for _ in range(9)] if M == 32 else [])
        turn = [0]

        def fn(at=at, wts=wts, bt=bt, ot=ot, M=M, turn=turn):
            turn[0] = (turn[0] + 1) % len(wts)
            hip.call("ttm_linear", hip.ptr(at), hip.BF16, hip.ptr(wts[turn[0]]), hip.BFP8B, 0, hip.ptr(bt), hip.BF16, hip.TILE,
                     hip.ptr(ot), hip.BF16, 1, 1, M, N, K, hip.ACT["gelu"], s)
        if M == 2048:
            out[nm] = Workload(nm, "mfma", 2.0 * M * N * K, "flop", fn,
                               "config 3: bf16 [2048,4096] x bfp8_b [4096,14336] + bias + GELU",
                               dict(host=(a, w, bias), dev=(at, wt, bt, ot)))
        else:
            nbytes = (K // 32) * (N // 32) * 1088 + 2 * M * K + 2 * M * N + 2 * N
            out[nm] = Workload(nm, "hbm", nbytes, "bytes", fn,
                               "config 3 decode: bf16 [32,4096] x bfp8_b [4096,14336] + bias + GELU (weight streaming; ten weight "
                               "copies cycled, so each launch reads HBM)",
                               dict(flop=2.0 * M * N * K))
    if "sdpa_decode32" in names:
        B, H, Hkv, S, D = 32, 32, 8, 2048, 128
        q = datagen.randn((1, B, H, D), seed=1, dtype=torch.bfloat16).to(dev)
        kv = [datagen.randn((B, Hkv, S, D), seed=2 + i, dtype=torch.bfloat16).to(dev) for i in range(2)]
        qt, o = torch.empty(B * 32 * D, dtype=torch.bfloat16, device=dev), torch.empty(B * 32 * D, dtype=torch.bfloat16, device=dev)
        hip.call("ttm_tilize", hip.ptr(q), hip.ptr(qt), B, H, D, 2, s)
        kvt = [torch.empty_like(t) for t in kv]
        for t, tt in zip(kv, kvt):
            hip.call("ttm_tilize", hip.ptr(t), hip.ptr(tt), B * Hkv, S, D, 2, s)
        cur = torch.full((B,), S - 1, dtype=torch.int32, device=dev)
        torch.cuda.synchronize()
        del kv
        # the two caches of one layer (268 MB) are about the size of the 256 MB last-level cache: three pairs are cycled
        # (805 MB), as the layers of a model would be, so that every launch reads HBM
        caches = [kvt] + [[t.clone() for t in kvt] for _ in range(2)]
        dturn = [0]

        def dfn(qt=qt, caches=caches, cur=cur, o=o, B=B, H=H, Hkv=Hkv, S=S, D=D, dturn=dturn):
            dturn[0] = (dturn[0] + 1) % len(caches)
            kc, vc = caches[dturn[0]]
            hip.call("ttm_sdpa_decode", hip.ptr(qt), hip.ptr(kc), hip.ptr(vc), hip.ptr(cur), None, 1, None, 0, 0, 0,
                     hip.ptr(o), hip.BF16, B, H, Hkv, S, D, 1, 0.0, s)
        out["sdpa_decode32"] = Workload(
            "sdpa_decode32", "hbm", 2 * B * Hkv * S * D * 2 + 2 * B * H * D * 2, "bytes", dfn,
            "decode attention: 32 users x 32 heads (8 kv heads) x 1 token over a full 2048-position bf16 KV cache (three cache "
            "pairs cycled, so each launch reads HBM)",
            dict(keep=(qt, caches, cur, o)))
    for nm, window in (("sdpa2048", -1), ("sdpa2048_window128", 128)):
        if nm not in names:
            continue
        B, Hq, Hkv, S, D = 1, 32, 8, 2048, 128
        qkv = [datagen.randn((B, h, S, D), seed=5 + i, dtype=torch.bfloat16).to(dev) for i, h in enumerate((Hq, Hkv, Hkv))]
        tiles = [torch.empty_like(t) for t in qkv]
        for t, tt, h in zip(qkv, tiles, (Hq, Hkv, Hkv)):
            hip.call("ttm_tilize", hip.ptr(t), hip.ptr(tt), B * h, S, D, 2, s)
        o = torch.empty_like(tiles[0])
        torch.cuda.synchronize()
        del qkv
        # full causal pass: dense count, the convention of the decoder-layer figure (about half of it is computed);
        # windowed pass: the visible (query, key) pairs only, sum_i min(i + 1, w), so the fraction is not flattered
        # FLOPs of the visible (query, key) pairs only: the causal triangle S (S + 1) / 2, or sum_i min(i + 1, w) under a
        # window; the dense count 4 B Hq S^2 D (the convention of the decoder-layer figure) is reported beside it
        visible = sum(min(i + 1, window) for i in range(S)) if window >= 0 else S * (S + 1) // 2
        out[nm] = Workload(
            nm, "mfma", 2.0 * 2 * B * Hq * visible * D, "flop",
            lambda tiles=tiles, o=o, window=window, B=B, Hq=Hq, Hkv=Hkv, S=S, D=D: hip.call(
                "ttm_sdpa_windowed", hip.ptr(tiles[0]), hip.ptr(tiles[1]), hip.ptr(tiles[2]), None, 1, 1, hip.ptr(o), hip.BF16, B, Hq, Hkv,
                S, S, D, 1, 0.0, 0, window, None, s),
            "config 5 attention alone: causal SDPA, 32 query / 8 kv heads, 2048 tokens, head_dim 128" +
            (" (FLOPs of the causal triangle only)" if window < 0 else ", sliding window of %d keys (FLOPs of the visible pairs only)" % window),
            dict(keep=(tiles, o), dense_flop=2.0 * 2 * B * Hq * S * S * D))
    # bandwidth class of the layer: RMSNorm, softmax and a last-dim reduction at config-5 sizes, SiLU(gate) * up at config 4's
    if "rmsnorm2048" in names:
        R_, C_ = 2048, 4096
        xr = datagen.randn((R_, C_), seed=21, dtype=torch.bfloat16).to(dev)
        wr = (1.0 + 0.02 * datagen.randn((1, C_), seed=22)).to(torch.bfloat16).to(dev)
        xt_, wt_ = torch.empty_like(xr), torch.zeros(32 * C_, dtype=torch.bfloat16, device=dev)
        hip.call("ttm_tilize", hip.ptr(xr), hip.ptr(xt_), 1, R_, C_, 2, s)
        hip.call("ttm_tilize", hip.ptr(wr), hip.ptr(wt_), 1, 1, C_, 2, s)
        yt_ = torch.empty_like(xt_)
        out["rmsnorm2048"] = Workload(
            "rmsnorm2048", "hbm", 2 * R_ * C_ * 2 + C_ * 2, "bytes",
            lambda xt_=xt_, wt_=wt_, yt_=yt_, R_=R_, C_=C_: hip.call("ttm_rms_norm", hip.ptr(xt_), hip.ptr(wt_), hip.TILE, None, hip.TILE, hip.ptr(yt_),
                                                       hip.BF16, 1, R_, C_, 1e-5, s),
            "config 5 RMSNorm: bf16 [2048,4096] tiles, weight [4096], eps 1e-5", dict(keep=(xt_, wt_, yt_)))
    if "softmax65536" in names or "reduce65536" in names:
        R_, C_ = 32 * 2048, 2048
        xs = (3.0 * datagen.randn((R_, C_), seed=23)).to(dev)
        xt_ = torch.empty_like(xs)
        hip.call("ttm_tilize", hip.ptr(xs), hip.ptr(xt_), 1, R_, C_, 4, s)
        torch.cuda.synchronize()
        del xs
        if "softmax65536" in names:
            yt_ = torch.empty_like(xt_)
            out["softmax65536"] = Workload(
                "softmax65536", "hbm", 2 * R_ * C_ * 4, "bytes",
                lambda xt_=xt_, yt_=yt_, R_=R_, C_=C_: hip.call("ttm_softmax_lastdim", hip.ptr(xt_), hip.ptr(yt_), hip.F32, 1, R_, C_, s),
                "config 5 attention scores if left unfused: softmax over the last dim of fp32 [32 x 2048, 2048] tiles",
                dict(keep=(xt_, yt_)))
        if "reduce65536" in names:
            rt_ = torch.empty(R_ * 32, dtype=torch.float32, device=dev)
            out["reduce65536"] = Workload(
                "reduce65536", "hbm", R_ * C_ * 4 + R_ * 4, "bytes",
                lambda xt_=xt_, rt_=rt_, R_=R_, C_=C_: hip.call("ttm_reduce_lastdim", 0, hip.ptr(xt_), hip.ptr(rt_), hip.F32, 1, R_, C_, s),
                "sum over the last dim of fp32 [32 x 2048, 2048] tiles (one value per row)", dict(keep=(xt_, rt_)))
    if "silu_mul512" in names:
        import numpy as np
        R_, C_ = 512, 14336
        g_ = datagen.randn((R_, C_), seed=24, dtype=torch.bfloat16).to(dev)
        u_ = datagen.randn((R_, C_), seed=25, dtype=torch.bfloat16).to(dev)
        gt_, ut_ = torch.empty_like(g_), torch.empty_like(u_)
        hip.call("ttm_tilize", hip.ptr(g_), hip.ptr(gt_), 1, R_, C_, 2, s)
        hip.call("ttm_tilize", hip.ptr(u_), hip.ptr(ut_), 1, R_, C_, 2, s)
        ot_ = torch.empty_like(gt_)
        shp = np.array([R_, C_], dtype=np.int64)
        out["silu_mul512"] = Workload(
            "silu_mul512", "hbm", 3 * R_ * C_ * 2, "bytes",
            lambda gt_=gt_, ut_=ut_, ot_=ot_, shp=shp: hip.call("ttm_eltwise_binary", 1, hip.ptr(gt_), shp.ctypes.data, hip.ptr(ut_),
                                                                shp.ctypes.data, hip.ptr(ot_), shp.ctypes.data, 2, hip.BF16, hip.TILE, s),
            "config 4 SiLU(gate) * up: bf16 [512,14336] tiles, two reads and one write (the SiLU itself sits in the gate "
            "projection's epilogue)", dict(keep=(gt_, ut_, ot_, shp)))
    # whole programs through the runtime boundary (flatbuffer -> submit -> wait)
    for nm in ("decode32", "decode32_traced"):
        if nm not in names:
            continue
        from ttmlir_amd import programs, runtime as rt
        users, hidden, n_q, n_kv, hd, ffn, max_seq, pos = 32, 4096, 32, 8, 128, 14336, 2048, 2047
        binary = rt.Binary.load_from_memory(programs.decode_layer(users, hidden, n_q, n_kv, hd, ffn, max_seq, trace=nm.endswith("traced"),
                                                                  host_inputs=False))
        main = binary.get_num_programs() - 1
        r16 = lambda shape, seed, scale=1.0: (datagen.randn(shape, seed=seed, dtype=torch.float32) * scale).to(torch.bfloat16)
        wshapes = [(hidden,), (hidden, n_q * hd), (hidden, n_kv * hd), (hidden, n_kv * hd), (n_q * hd, hidden), (hidden,), (hidden, ffn),
                   (hidden, ffn), (ffn, hidden)]
        tins = [r16((users, hidden), 1), r16((1, 1, 1, hd), 2), r16((1, 1, 1, hd), 3), torch.tensor([pos], dtype=torch.int32),
                torch.full((users,), pos, dtype=torch.int32), r16((users, n_kv, max_seq, hd), 4), r16((users, n_kv, max_seq, hd), 5)]
        tins += [r16(sh, 10 + i, 0.02) for i, sh in enumerate(wshapes)]
        rdev = rt.open_mesh_device()
        rins = [rt.to_layout(rt.from_torch(t), rdev, rt.get_layout(binary, main, i), retain=True) for i, t in enumerate(tins)]
        del tins
        # bytes one step must move: block-float weights once, both caches up to the current position, activations
        wbytes = sum((a // 32) * (b // 32) * 1088 for a, b in (wshapes[1], wshapes[2], wshapes[3], wshapes[4], wshapes[6], wshapes[7]))
        wbytes += (ffn // 32) * (hidden // 32) * 576
        nbytes = wbytes + 2 * users * n_kv * (pos + 1) * hd * 2

        # a step is one submit; steps follow each other on the device's stream as the layers of a model would (each reads the
        # caches the previous one wrote), and the timed region ends with a device-wide wait.  `latency` is one submit
        # followed by a wait of its own
        def run(binary=binary, rins=rins, rdev=rdev, main=main):
            rt.submit(rdev, binary, main, rins)

        def run_and_wait(binary=binary, rins=rins, rdev=rdev, main=main):
            rt.wait(rt.submit(rdev, binary, main, rins))

        out[nm] = Workload(nm, "hbm", nbytes, "bytes", run,
                           "Llama-3-8B decoder layer, one token for 32 users at position 2047 (weights bfp8_b / bfp4_b, bf16 KV cache "
                           "updated in place), one submit" + (" replaying a captured HIP graph" if nm.endswith("traced") else ""),
                           dict(sync=True, steps=50, latency=run_and_wait, keep=(rdev, rins, binary)))
    for nm in ("mlp512", "decoder2048"):
        if nm not in names:
            continue
        from ttmlir_amd import programs, runtime as rt
        bfl = lambda t: t.to(torch.bfloat16)
        if nm == "mlp512":
            d = datagen.c4_mlp()
            binary = rt.Binary.load_from_memory(programs.c4_mlp())
            tins = [d["x"], d["norm_w"], bfl(d["wg"]), bfl(d["wu"]), bfl(d["wd"])]
            flop, desc = 180388626432.0, "config 4: Llama MLP block, 512 tokens (RMSNorm, gate/up bfp8_b, SiLU*up, down bfp4_b), one submit"
        else:
            d = datagen.c5_decoder()
            binary = rt.Binary.load_from_memory(programs.c5_decoder())
            tins = [d["x"], d["attn_norm_w"], bfl(d["wq"]), bfl(d["wk"]), bfl(d["wv"]), bfl(d["wo"]), d["mlp_norm_w"], bfl(d["wg"]),
                    bfl(d["wu"]), bfl(d["wd"])]
            flop = 893353197568.0 + 68719476736.0
            desc = "config 5: Llama-3-8B decoder layer, batch 1, seq 2048 prefill (dense attention FLOPs counted), one submit"
        rdev = rt.open_mesh_device()
        rins = [rt.to_layout(rt.from_torch(t), rdev, rt.get_layout(binary, 1, i), retain=True) for i, t in enumerate(tins)]
        del d, tins

        def run(binary=binary, rins=rins, rdev=rdev):
            for o in rt.submit(rdev, binary, 1, rins):
                rt.deallocate_tensor(o, force=True)      # back to the stream-ordered pool; the next step may reuse it

        def run_and_wait(binary=binary, rins=rins, rdev=rdev):
            outs = rt.submit(rdev, binary, 1, rins)
            rt.wait(outs)
            for o in outs:
                rt.deallocate_tensor(o, force=True)

        out[nm] = Workload(nm, "mfma", flop, "flop", run, desc, dict(sync=True, latency=run_and_wait, keep=(rdev, rins, binary)))
    return out


# HBM bytes per launch of each workload's kernel, from two rocprofv3 --pmc runs (FETCH_SIZE, then WRITE_SIZE) scaled by
# what the same counters read for the plain copy kernel of known size (factors 1.9998 and 0.9999); these are measured
# constants of the committed kernels, not computed here (profiles/bench_kernels_hbm_traffic_pmc.md holds the table and
# the commands).  linear2048 is a two-pass launch: 181.9 MB for the pass that writes the weights as bf16 fragment images
# plus 447.6 MB for the matrix pass (every XCD's L2 fetches the activations and its share of the images again).  Each
# figure belongs to one version of a kernel source file: it is reported only while that file still has the content it
# was measured on (first 12 hex digits of its SHA-1), else `traffic` is null and `traffic_source` says so.
MEASURED_TRAFFIC_BYTES = {
    "linear2048": (629.5e6, "ttm_linear.hip"), "linear32": (65.6e6, "ttm_linear.hip"), "pack_bfp8": (340.4e6, "ttm_bfp.hip"),
    "unpack_bfp8": (340.1e6, "ttm_bfp.hip"), "pack_bfp4": (306.2e6, "ttm_bfp.hip"), "unpack_bfp4": (306.6e6, "ttm_bfp.hip"),
    "tilize_f32": (537.3e6, "ttm_layout.hip"), "untilize_f32": (537.0e6, "ttm_layout.hip"), "copy": (536.9e6, "ttm_layout.hip"),
    "sdpa_decode32": (270.3e6, "ttm_decode.hip"), "sdpa2048": (42.3e6, "ttm_sdpa.hip"), "rmsnorm2048": (34.0e6, "ttm_rowwise.hip"),
    "softmax65536": (1073.8e6, "ttm_rowwise.hip"), "reduce65536": (545.2e6, "ttm_rowwise.hip"), "silu_mul512": (44.2e6, "ttm_eltwise.hip"),
}
MEASURED_ON = {"ttm_linear.hip": ("875295d3c654",), "ttm_bfp.hip": ("cdf35c7592c1",), "ttm_layout.hip": ("a6cf1c428342",),
               "ttm_decode.hip": ("3bd99843ac98",), "ttm_rowwise.hip": ("0819544c7ff3",), "ttm_eltwise.hip": ("62019175607e",),
               "ttm_sdpa.hip": ("3c1e7f59da68",)}
TRAFFIC_HOW = ("rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE (two runs), KiB per dispatch scaled by what the same counters "
               "read for the 256 MiB copy kernel; profiles/bench_kernels_hbm_traffic_pmc.md")


def measured_traffic(name):
    """(bytes per launch, where the figure comes from) or (None, why there is none)."""
    import hashlib
    entry_ = MEASURED_TRAFFIC_BYTES.get(name)
    if entry_ is None:
        return None, "not measured for this workload"
    nbytes, source = entry_
    try:
        with open(os.path.join(ROOT, "tt-mlir_amd", "csrc", source), "rb") as f:
            digest = hashlib.sha1(f.read()).hexdigest()[:12]
    except OSError:
        return None, "kernel source %s not found" % source
    if digest in MEASURED_ON.get(source, ()):
        return nbytes, TRAFFIC_HOW
    return None, "%s has changed since its kernels' counters were read" % source


def roofline(w, kernel_ms):
    if w.bound == "hbm":
        achieved = w.work / (kernel_ms * 1e-3) / 1e9
        peak, unit = HBM_PEAK_GBS, "GB/s"
    else:
        achieved = w.work / (kernel_ms * 1e-3) / 1e12
        peak, unit = MFMA_BF16_PEAK_TFLOPS, "TFLOP/s"
    traffic, how = measured_traffic(w.name)
    r = {"bound": w.bound, "achieved": round(achieved, 2), "peak": peak, "unit": unit,
         "frac": round(achieved / peak, 4), "traffic": traffic, "traffic_source": how, "kernel_us": round(kernel_ms * 1e3, 2),
         "algorithmic_work": w.work, "work_unit": w.unit_work}
    if "dense_flop" in w.extra:   # attention: the dense count beside the FLOPs of the visible pairs that `frac` is made of
        dense = w.extra["dense_flop"] / (kernel_ms * 1e-3) / 1e12
        r["dense_counted"] = {"achieved": round(dense, 2), "frac": round(dense / peak, 4), "work": w.extra["dense_flop"]}
    return r


def cpu_baseline_linear(orc, datagen, budget_rows=512):
    """The CPU path (scalar f32 loops, one thread) on a row sample of config 3, M=2048."""
    import numpy as np
    import torch
    a, w, bias = datagen.c3_linear(2048)
    weff = orc.bfp_unpack(orc.bfp_pack(w.numpy(), 8), w.shape, 8)      # the weights the device multiplies
    rows = a[:budget_rows].float().numpy()
    K, N = w.shape
    orc.set_threads(1)
    t0 = time.perf_counter()
    y = orc.linear(rows, weff, bias.float().numpy(), "gelu", rowstream=True)
    dt = time.perf_counter() - t0
    one = 2.0 * budget_rows * N * K / dt / 1e12
    cores = min(16, orc.max_threads())
    orc.set_threads(cores)
    big = a[:budget_rows * 4].float().numpy()
    t0 = time.perf_counter()
    orc.linear(big, weff, bias.float().numpy(), "gelu", rowstream=True)
    dtn = time.perf_counter() - t0
    orc.set_threads(1)
    alln = 2.0 * budget_rows * 4 * N * K / dtn / 1e12
    return {"value": round(one, 6), "unit": "TFLOP/s", "cores": 1, "kind": "port",
            "sample": "oracle scalar f32 linear+bias+GELU on rows 0..%d of config 3 (M=2048, K=4096, N=14336), "
                      "dequantised bfp8_b weights, %.1f s" % (budget_rows - 1, dt),
            "all_cores": {"value": round(alln, 6), "cores": cores, "rows": budget_rows * 4, "seconds": round(dtn, 2)}}, y


def cpu_baseline_pack(orc, datagen, rows=8192):
    x = datagen.c2_outliers(rows, 8192, seed=0).numpy()
    orc.set_threads(1)
    t0 = time.perf_counter()
    orc.bfp_pack(x, 8)
    dt = time.perf_counter() - t0
    nbytes = rows * 8192 * 4 + (rows // 32) * 256 * 1088
    return {"value": round(nbytes / dt / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "oracle bfp8_b pack of %d x 8192 fp32 rows of config 2, %.2f s" % (rows, dt)}


def cpu_baseline_secondary(orc, datagen, name):
    """The CPU restatement (one thread, scalar loops) on a bounded sample of a secondary workload, in the workload's own
    unit: algorithmic bytes (or FLOP) of the sample over the time it took.  None for workloads without one function to time
    (whole programs, the plain copy)."""
    import numpy as np
    rng = np.random.default_rng(0)
    orc.set_threads(1)

    def timed(fn):
        t0 = time.perf_counter()
        fn()
        return time.perf_counter() - t0

    def entry_(work, dt, unit, sample):
        scale = 1e12 if unit == "TFLOP/s" else 1e9
        return {"value": round(work / dt / scale, 6), "unit": unit, "cores": 1, "kind": "port", "sample": "%s, %.2f s" % (sample, dt)}

    if name in ("pack_bfp8", "pack_bfp4", "unpack_bfp8", "unpack_bfp4"):
        fmt, rows = (8 if name.endswith("8") else 4), 2048
        x = datagen.c2_outliers(rows, 8192, seed=0).numpy()
        nbytes = rows * 8192 * 4 + (rows // 32) * 256 * orc.bfp_tile_bytes(fmt)
        if name.startswith("pack"):
            return entry_(nbytes, timed(lambda: orc.bfp_pack(x, fmt)), "GB/s", "oracle bfp%d_b pack of %d x 8192 fp32 rows of config 2" % (fmt, rows))
        packed = orc.bfp_pack(x, fmt)
        return entry_(nbytes, timed(lambda: orc.bfp_unpack(packed, x.shape, fmt)), "GB/s", "oracle bfp%d_b unpack of %d x 8192 rows of config 2" % (fmt, rows))
    if name in ("tilize_f32", "untilize_f32"):
        rows = 4096
        x = rng.standard_normal((rows, 8192), dtype=np.float32)
        if name == "tilize_f32":
            return entry_(2 * x.nbytes, timed(lambda: orc.tilize(x)), "GB/s", "oracle tilize of %d x 8192 fp32 rows of config 2" % rows)
        t = orc.tilize(x)
        return entry_(2 * x.nbytes, timed(lambda: orc.untilize(t, x.shape)), "GB/s", "oracle untilize of %d x 8192 fp32 rows of config 2" % rows)
    if name == "linear32":
        a, w, bias = datagen.c3_linear(32)
        weff = orc.bfp_unpack(orc.bfp_pack(w.numpy(), 8), w.shape, 8)
        an, bn = a.float().numpy(), bias.float().numpy()
        K, N = w.shape
        nbytes = (K // 32) * (N // 32) * 1088 + 2 * 32 * K + 2 * 32 * N + 2 * N
        return entry_(nbytes, timed(lambda: orc.linear(an, weff, bn, "gelu", rowstream=True)), "GB/s",
                      "oracle scalar f32 linear+bias+GELU, all 32 rows of config 3 (weight bytes counted as bfp8_b tiles)")
    if name == "sdpa2048":
        q = rng.standard_normal((1, 1, 2048, 128), dtype=np.float32)
        k = rng.standard_normal((1, 1, 2048, 128), dtype=np.float32)
        v = rng.standard_normal((1, 1, 2048, 128), dtype=np.float32)
        flop = 4.0 * 2048 * 2048 * 128 / 2
        return entry_(flop, timed(lambda: orc.sdpa(q, k, v, None, is_causal=True)), "TFLOP/s", "oracle causal SDPA, one of the 32 heads of config 5 (FLOPs of the causal triangle)")
    if name == "sdpa_decode32":
        users, H, Hkv, S, D = 4, 32, 8, 2048, 128
        q = rng.standard_normal((1, users, H, D), dtype=np.float32)
        k = rng.standard_normal((users, Hkv, S, D), dtype=np.float32)
        v = rng.standard_normal((users, Hkv, S, D), dtype=np.float32)
        pos = np.full((users,), S - 1, dtype=np.int32)
        nbytes = 2 * users * Hkv * S * D * 2 + 2 * users * H * D * 2
        return entry_(nbytes, timed(lambda: orc.sdpa_decode(q, k, v, cur_pos=pos)), "GB/s", "oracle decode attention, 4 of the 32 users (cache bytes counted as bf16)")
    if name == "rmsnorm2048":
        x = rng.standard_normal((2048, 4096), dtype=np.float32)
        w = rng.standard_normal((4096,), dtype=np.float32)
        return entry_(2 * 2048 * 4096 * 2 + 4096 * 2, timed(lambda: orc.rms_norm(x, w, None, 1e-5)), "GB/s", "oracle RMSNorm of [2048, 4096] (bytes counted as bf16)")
    if name == "softmax65536":
        x = rng.standard_normal((4096, 2048), dtype=np.float32)
        return entry_(2 * x.nbytes, timed(lambda: orc.softmax(x, -1)), "GB/s", "oracle softmax over 4096 of the 65536 rows of 2048 fp32")
    if name == "reduce65536":
        x = rng.standard_normal((8192, 2048), dtype=np.float32)
        return entry_(x.nbytes + 8192 * 32 * 4, timed(lambda: orc.reduce("sum", x, -1, True)), "GB/s", "oracle sum over 8192 of the 65536 rows of 2048 fp32")
    if name == "silu_mul512":
        g = rng.standard_normal((512, 14336), dtype=np.float32)
        u = rng.standard_normal((512, 14336), dtype=np.float32)
        return entry_(3 * 512 * 14336 * 2, timed(lambda: orc.binary("multiply", orc.round_bf16(orc.unary("silu", g)), u)), "GB/s",
                      "oracle SiLU(gate) * up on [512, 14336] (bytes counted as bf16)")
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="linear2048")
    ap.add_argument("--secondary", default="pack_bfp8,unpack_bfp8,pack_bfp4,unpack_bfp4,tilize_f32,untilize_f32,copy,linear32,sdpa_decode32,sdpa2048,rmsnorm2048,"
                                           "softmax65536,reduce65536,silu_mul512,mlp512,decoder2048,decode32,decode32_traced")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-settle", action="store_true",
                    help="skip the 0.3 s of untimed launches in front of every measurement (counter collection runs, where "
                         "every dispatch is expensive)")
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="kernel-variant option passed to ttm_set_option before anything runs (e.g. linear_two_pass=1)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (one MI355X per box); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import torch
    entry.load_package()
    from ttmlir_amd import hip, datagen
    hip.lib()
    for opt in args.option:
        name, _, value = opt.partition("=")
        hip.set_option(name, int(value))
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    stream = hip.current_stream()
    sec_names = [n for n in args.secondary.split(",") if n and n != args.workload and n != "none"]
    wl = make_workloads(torch, hip, datagen, dev, [args.workload] + sec_names)
    if args.workload not in wl:
        raise SystemExit("unknown workload " + args.workload)

    def measure(w, steps, warmup):
        # clocks settle only after some tens of milliseconds of load: keep the device busy for about 0.3 s before
        # the `warmup` untimed steps, so that short default runs measure the steady state
        t_end = time.perf_counter() + (0.0 if args.no_settle else 0.3)
        while time.perf_counter() < t_end:
            for _ in range(8):
                w.fn()
            torch.cuda.synchronize()
        for _ in range(warmup):
            w.fn()
        ms = _wall_time(torch, w.fn, steps)                    # timed region: exactly `steps` launches
        if w.extra.get("sync"):                                # whole programs run on the runtime's own stream: wall time of the steps
            return ms, ms
        kms = _events_time(hip, stream, w.fn, steps)           # HIP events on the launch stream
        return ms, kms

    prim = wl[args.workload]
    ms, kms = measure(prim, args.steps, args.warmup)
    rl = roofline(prim, kms)
    if prim.bound == "mfma":
        value, unit, metric = prim.work / (ms * 1e-3) / 1e12, "TFLOP/s", "bfp8_b matmul TFLOP/s"
    else:
        value, unit, metric = prim.work / (ms * 1e-3) / 1e9, "GB/s", prim.name + " GB/s"
    secondary = []
    for n in sec_names:
        w = wl[n]
        heavy = bool(w.extra.get("sync"))
        sms, skms = measure(w, w.extra.get("steps", 5) if heavy else max(10, args.steps // 2), 2 if heavy else max(3, args.warmup // 2))
        r = roofline(w, skms)
        if w.bound == "hbm" and not heavy and w.work < 200e6:
            # small tensors: a launch of a few microseconds is mostly ramp; the plain copy kernel moving the same number of
            # bytes (half read, half written) is the ceiling to hold the figure against
            half = int(w.work // 2) // 16 * 16
            cx = torch.empty(half, dtype=torch.uint8, device=dev)
            cy = torch.empty_like(cx)
            cfn = lambda cx=cx, cy=cy, half=half: hip.call("ttm_copy_kernel", hip.ptr(cx), hip.ptr(cy), half, stream)
            for _ in range(20):
                cfn()
            cms = _events_time(hip, stream, cfn, 50)
            r["copy_of_same_bytes"] = {"kernel_us": round(cms * 1e3, 2), "achieved": round(2 * half / (cms * 1e-3) / 1e9, 2), "unit": "GB/s"}
            del cx, cy
        entry_ = {"workload": n, "desc": w.desc, "ms_per_step": round(sms, 5), "roofline": r}
        if "latency" in w.extra:   # one step with a wait of its own (launch and wake-up latencies included)
            entry_["latency_ms"] = round(_wall_time(torch, w.extra["latency"], 10), 5)
        secondary.append(entry_)

    result = {
        "metric": metric, "value": round(value, 3), "unit": unit, "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16 x bfp8_b -> f32 accumulate" if "linear" in prim.name else "u8/f32 bits",
        "data": "synthetic",
        "config": {"workload": prim.desc, "name": prim.name, "device": hip.device_name()},
        "roofline": rl, "secondary": secondary,
    }
    if prim.name == "linear2048":
        # the vendor library's plain bf16 x bf16 GEMM at the same M, N, K (weights already bf16: no block-float decode, no
        # bias, no GELU), as a reference point for what the matrix cores sustain on this device at this shape
        xa = torch.randn(2048, 4096, device=dev).to(torch.bfloat16)
        xw = (0.02 * torch.randn(4096, 14336, device=dev)).to(torch.bfloat16)
        lib_w = Workload("library_gemm", "mfma", prim.work, "flop", lambda: torch.matmul(xa, xw), "torch.matmul bf16 x bf16")
        lms, _ = measure(lib_w, max(10, args.steps // 2), max(3, args.warmup // 2))
        result["library_gemm"] = {"what": "torch.matmul bf16 [2048,4096] x bf16 [4096,14336] (vendor BLAS, no decode / bias / GELU)",
                                  "ms_per_step": round(lms, 5), "value": round(prim.work / (lms * 1e-3) / 1e12, 1), "unit": "TFLOP/s"}
        # The matrix cores run against the board's power limit: the shader clock under this load is well below the 2400 MHz
        # that the published peak assumes, and it depends on the operand values.  Reported: the clock while this kernel and
        # while the vendor GEMM loop on the same operands, and the same launches on all-zero operands (no switching in the
        # multipliers: the clock stays at its maximum), which separates what the kernel's schedule costs from what the
        # power limit costs.
        if not args.no_settle:
            sclk, nsamp, loop_ms = sample_sclk(torch, prim.fn)
            lclk, _, lloop = sample_sclk(torch, lib_w.fn)
            at, wt, bt, ot = prim.extra["dev"]
            keep = (at.clone(), wt.clone())
            at.zero_(), wt.zero_()
            zclk, _, zloop = sample_sclk(torch, prim.fn)
            xa.zero_(), xw.zero_()
            zlclk, _, zlloop = sample_sclk(torch, lib_w.fn)
            at.copy_(keep[0]), wt.copy_(keep[1])
            del keep
            prim.fn()                                   # the output checked below comes from the real operands again
            torch.cuda.synchronize()
            result["clock"] = {
                "sclk_mhz_max": 2400, "sclk_mhz_this_kernel": sclk, "loop_ms_this_kernel": round(loop_ms, 5), "samples": nsamp,
                "sclk_mhz_library_gemm": lclk, "loop_ms_library_gemm": round(lloop, 5),
                "zero_operands": {"sclk_mhz_this_kernel": zclk, "loop_ms_this_kernel": round(zloop, 5),
                                  "sclk_mhz_library_gemm": zlclk, "loop_ms_library_gemm": round(zlloop, 5)},
                "what": "shader clock (the driver's pp_dpm_sclk) while the launch is repeated back to back for 1.2 s, and the same with all-zero "
                        "operands; loop_ms includes launch gaps"}
        del xa, xw
    if not args.no_cpu_baseline:
        orc = entry.load_oracle()
        if "linear" in prim.name:
            cb, y_cpu = cpu_baseline_linear(orc, datagen)
            result["cpu_baseline"] = cb
            # the same rows from the GPU output, as a last sanity check of what was timed
            if prim.name == "linear2048":
                import numpy as np
                at, wt, bt, ot = prim.extra["dev"]
                o = torch.empty((2048, 14336), dtype=torch.bfloat16, device=dev)
                hip.call("ttm_untilize", hip.ptr(ot), hip.ptr(o), 1, 2048, 14336, 2, stream)
                torch.cuda.synchronize()
                g = o[: y_cpu.shape[0]].float().cpu().numpy()
                result["check"] = {"rows": int(y_cpu.shape[0]),
                                   "max_abs_err_vs_cpu": float(np.max(np.abs(g - orc.round_bf16(y_cpu))))}
        else:
            result["cpu_baseline"] = cpu_baseline_pack(orc, datagen)
        result["cpu_baseline_pack_bfp8"] = cpu_baseline_pack(orc, datagen)
        for e in secondary:   # the same path on the host cores, on a bounded sample of every kernel workload
            cb = cpu_baseline_secondary(orc, datagen, e["workload"])
            if cb is not None:
                e["cpu_baseline"] = cb
    print(json.dumps(result))


if __name__ == "__main__":
    main()
