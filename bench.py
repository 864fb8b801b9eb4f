#!/usr/bin/env python3
"""Benchmark of the batched-decode hot path on one MI355X.

Workload (BASELINE.json north star): LLaMA-2-7B-shaped decoder (32 layers, hidden 4096, 32 MHA
heads, head_dim 128, FFN 11008, vocab 32000), random-init N(0,0.02) weights quantized to Q4_0
(token embedding and output head Q8_0, the rule of config 1), F16 paged KV (block 16) pre-filled
with N(0,1), 32 ragged sequences with contexts lognormal(median 1024, sigma 0.6) clipped to
[64, 4096] (seed 0), block tables a seeded permutation of the physical blocks. A step is one
greedy decode step of all 32 sequences (pack -> 32 layers -> head -> argmax), replayed from a
hipGraph with inputs resident in HBM.

Prints ONE JSON line. The synthetic weights and KV contents are generated on the device by
libvexel_synth.so (benchmark support built next to the backend); no torch in this process.
"""
import argparse
import ctypes as C
import json
import math
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

CFG = dict(num_layers=32, hidden=4096, num_heads=32, num_kv_heads=32, head_dim=128, ffn=11008, vocab=32000)
BATCH = 32
BLOCK = 16


# HBM bytes per algorithmic byte of the attention launch, from rocprofv3 FETCH_SIZE / WRITE_SIZE counter runs
# scaled by a plain copy of known size (summary: profiles/paged_decode_attention_7b_x32_hbm_traffic.txt).
ATTN_TRAFFIC_PER_ALGORITHMIC_BYTE = 1.012
# the same for the step's four projection launches per layer at 32 rows
# (summary: profiles/decode_gemm_7b_q4_0_x32_issue_and_traffic_counters.txt)
GEMM_TRAFFIC_PER_ALGORITHMIC_BYTE = 1.23


def ragged_contexts(seed=0, n=BATCH):
    rng = np.random.default_rng(seed)
    ctx = np.exp(rng.normal(math.log(1024.0), 0.6, n))
    return [int(x) for x in np.clip(ctx, 64, 4096)]


def load_synth():
    """libvexel_synth.so: device-side generators of the synthetic weights and KV (benchmark support)."""
    path = os.path.join(ROOT, "vexel_amd", "libvexel_synth.so")
    if not os.path.exists(path):
        raise RuntimeError("%s is missing: run `python -m vexel_amd.build`" % path)
    s = C.CDLL(path)
    s.vxs_gaussian_quant.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_float, C.c_uint64]
    s.vxs_random_kquant.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_uint64]
    s.vxs_gaussian_f16.argtypes = [C.c_void_p, C.c_int64, C.c_float, C.c_uint64]
    s.vxs_plain_copy.argtypes = [C.c_void_p, C.c_void_p, C.c_int64]
    return s


def build_model(be, ctx, extra_tokens, layers, cfg=None, fmts=None, max_batch=None, arch=None, spare_tokens=0):
    """Synthetic model (7B-shaped Q4_0 unless cfg / fmts say otherwise) + pre-filled contexts, generated on the
    device. fmts: weight name (wq, wk, wv, wo, w1, w3, w2, head) -> VX_* format, "*" the default.
    arch: the switches of ModelRuntime.set_architecture plus "bias": "qkv" | "all" (small random bias vectors).
    spare_tokens: free pool blocks (and a free sequence slot) for one more sequence of that many tokens.
    -> (ModelRuntime, ids)"""
    from vexel_amd import lib
    from vexel_amd.runtime import ModelRuntime
    synth = load_synth()
    c = dict(cfg or CFG)
    c["num_layers"] = layers
    fmts = fmts or {"*": lib.VX_Q4_0, "head": lib.VX_Q8_0}
    fm = lambda name: fmts.get(name, fmts["*"])
    need_blocks = sum((L + extra_tokens + BLOCK - 1) // BLOCK + 1 for L in list(ctx) + ([spare_tokens] if spare_tokens else []))
    max_bps = (max(max(ctx), spare_tokens) + extra_tokens + BLOCK - 1) // BLOCK + 1
    mr = ModelRuntime(be, **c, pool_blocks=need_blocks, max_seqs=len(ctx) + (1 if spare_tokens else 0), max_blocks_per_seq=max_bps,
                      max_batch=max_batch or len(ctx), kv_fp16=True)
    seed = [0]
    arch = dict(arch or {})
    bias_kind = arch.pop("bias", None)
    if arch:
        mr.set_architecture(**arch)
    gelu_mlp = arch.get("mlp_type") == "gelu"

    def vec(n, mean):
        seed[0] += 1
        return (mean + 0.02 * np.random.default_rng(seed[0]).standard_normal(n)).astype(np.float32)

    def qbytes(n, k, fmt):
        return n * (k // 32) * (18 if fmt == lib.VX_Q4_0 else 34) if fmt in (lib.VX_Q4_0, lib.VX_Q8_0) else \
            n * (k // 256) * (144 if fmt == lib.VX_Q4_K else 210)

    def qfill(p, n, k, fmt):
        seed[0] += 1
        if fmt in (lib.VX_Q4_0, lib.VX_Q8_0):
            rc = synth.vxs_gaussian_quant(fmt, p, n * (k // 32), 0.02, seed[0])
        else:                                    # Q4_K / Q6_K: random valid super-blocks
            rc = synth.vxs_random_kquant(fmt, p, n * (k // 256), seed[0])
        if rc != 0:
            raise RuntimeError("synthetic weights failed: %d" % rc)
        return (fmt, p, n, k)

    def qw(n, k, fmt=lib.VX_Q4_0):
        p = be.alloc_permanent(qbytes(n, k, fmt) + 16)
        mr.adopt_device_buffer(p)
        return qfill(p, n, k, fmt)

    def qgroup(shapes):
        """The matrices one launch multiplies together (Q|K|V, gate|up), back to back in one buffer when they
        share format and width and every part starts on a 16-byte boundary; else one buffer each."""
        sizes = [qbytes(n, k, fmt) for n, k, fmt in shapes]
        if len({(k, fmt) for _, k, fmt in shapes}) != 1 or any(sz % 16 for sz in sizes):
            return [qw(n, k, fmt) for n, k, fmt in shapes]
        p = be.alloc_permanent(sum(sizes) + 16)
        mr.adopt_device_buffer(p)
        out, off = [], 0
        for (n, k, fmt), sz in zip(shapes, sizes):
            out.append(qfill(p + off, n, k, fmt))
            off += sz
        return out

    h, qd, kvd, f, v = c["hidden"], c["num_heads"] * c["head_dim"], c["num_kv_heads"] * c["head_dim"], c["ffn"], c["vocab"]
    layer_weights = []   # per layer: name -> (fmt, device pointer, n, k); kept on the runtime object for the GEMM timing
    mr.layer_weights = layer_weights
    ones = be.upload(np.ones(h, dtype=np.float32), permanent=True)
    mr.adopt_device_buffer(ones)
    for l in range(layers):
        wq, wk, wv = qgroup([(qd, h, fm("wq")), (kvd, h, fm("wk")), (kvd, h, fm("wv"))])
        wo = qw(h, qd, fm("wo"))
        w1, w3 = (qw(f, h, fm("w1")), None) if gelu_mlp else qgroup([(f, h, fm("w1")), (f, h, fm("w3"))])
        w2 = qw(h, f, fm("w2"))
        mr.set_layer(l, ones, ones, dict(wq=wq, wk=wk, wv=wv, wo=wo, w1=w1, w3=w3, w2=w2))
        layer_weights.append(dict(wq=wq, wk=wk, wv=wv, wo=wo, w1=w1, w3=w3, w2=w2))
        extras = {}
        if bias_kind in ("qkv", "all"):
            extras.update(wq_bias=vec(qd, 0.0), wk_bias=vec(kvd, 0.0), wv_bias=vec(kvd, 0.0))
        if bias_kind == "all":
            extras.update(wo_bias=vec(h, 0.0), w1_bias=vec(f, 0.0), w2_bias=vec(h, 0.0), attn_norm_bias=vec(h, 0.0))
        if arch.get("post_norms"):
            extras.update(post_attn_norm=vec(h, 1.0), post_ffn_norm=vec(h, 1.0))
        if extras:
            mr.set_layer_extras(l, **extras)
    emb_q = qw(v, h, lib.VX_Q8_0)
    emb = be.alloc_permanent(v * h * 4)
    mr.adopt_device_buffer(emb)
    be.dequantize(lib.VX_Q8_0, emb_q[1], emb, v * h)     # loader rule: token_embd kept in F32
    be.sync()
    mr.set_head(emb, ones, qw(v, h, fm("head")))
    # KV: every physical block of every layer holds N(0,1) halves
    per_block = 2 * BLOCK * kvd
    for l in range(layers):
        rc = synth.vxs_gaussian_f16(mr.kv_pool(l), need_blocks * per_block, 1.0, 1000 + l)
        if rc != 0:
            raise RuntimeError("vxs_gaussian_f16 failed: %d" % rc)
    rng = np.random.default_rng(0)
    perm = rng.permutation(need_blocks)
    ids, off = [], 0
    for i, L in enumerate(ctx):
        nb = (L + BLOCK - 1) // BLOCK
        mr.create_sequence(i + 1)
        mr.adopt_blocks(i + 1, perm[off:off + nb], L)
        off += nb
        ids.append(i + 1)
    return mr, ids


def attention_bytes(ctx_lens, c):
    """Algorithmic bytes of one ragged attention launch (one layer): K+V halves, block table, Q and out."""
    kvd, qd = c["num_kv_heads"] * c["head_dim"], c["num_heads"] * c["head_dim"]
    return sum(2 * L * kvd * 2 + ((L + BLOCK - 1) // BLOCK) * 4 + 2 * qd * 4 for L in ctx_lens)


def time_attention_kernel(be, mr, ctx_now, c, layers, reps, from_step=False):
    """Average duration of one launch of the ragged paged-attention kernel, HIP events on the backend stream,
    cycling over the layers' pools so every launch streams from HBM. The result is left in split form
    (out = NULL), as in the decode step, where the next kernel merges the splits."""
    b = len(ctx_now)
    qd = c["num_heads"] * c["head_dim"]
    q = be.upload(np.random.default_rng(1).standard_normal((b, qd)).astype(np.float32), permanent=True)
    out = be.alloc_permanent(b * qd * 4)
    own = []
    if from_step:
        # exactly the decode step's call: its block-table matrix, row indices and kv lengths (ctx_now), for
        # which the step's packing kernel has left the attention work list in the backend
        d_bt, d_rows, d_len = mr.step_buffers()
        got = be.download(d_len, (b,), np.int32)
        if list(got) != list(ctx_now):
            raise RuntimeError("the step's kv lengths are not the expected contexts")
    else:
        bts = np.zeros((b, mr.cfg.max_blocks_per_seq), dtype=np.int32)
        for i in range(b):
            t = mr.block_table(i + 1)
            bts[i, :len(t)] = t
        d_bt = be.upload(bts, permanent=True)
        d_len = be.upload(np.array(ctx_now, dtype=np.int32), permanent=True)
        d_rows = None
        own = [d_bt, d_len]
    scale = 1.0 / math.sqrt(c["head_dim"])
    cap = mr.cfg.max_blocks_per_seq * BLOCK

    def run(n):
        for i in range(n):
            be.sdpa_paged_decode_ragged(q, mr.kv_pool(i % layers), True, d_bt, d_len, None, b, mr.cfg.max_blocks_per_seq,
                                        BLOCK, c["num_heads"], c["num_kv_heads"], c["head_dim"], scale, cap,
                                        table_rows=d_rows)
    run(layers)
    be.sync()
    be.timer_start()
    run(reps)
    ms = be.timer_stop_ms()
    for p in [q, out] + own:
        be.free(p)
    return ms / reps


def cpu_baseline(be, mr, ctx, c, sample_layers=2, head_rows=2000, threads=1):
    """The reference CPU path (our C restatement, one core: the reference parallelises matmuls over M
    only and decodes one sequence at a time, cpu.go:856-870, decode.go:642-650) timed on a bounded
    sample: `sample_layers` layers + `head_rows` lm_head rows for one sequence, scaled to a full token.
    The random bytes that stand for the weights are not the GPU run's weights: values differ, timing does not
    depend on them. threads > 1: every matmul's weight rows are cut into that many slices computed side by side
    (NOT what the reference does; shown beside the one-core figure for scale)."""
    from concurrent.futures import ThreadPoolExecutor
    from oracle import numerics as nx
    L = ctx[0]
    hd, qd, kvd, f = c["hidden"], c["num_heads"] * c["head_dim"], c["num_kv_heads"] * c["head_dim"], c["ffn"]
    rng = np.random.default_rng(2)
    rb = lambda k: k // 32 * 18
    w = {}
    # weights of the sampled layers: random Q4_0 bytes of the real shapes (timing only)
    for name, (n, k) in dict(wq=(qd, hd), wk=(kvd, hd), wv=(kvd, hd), wo=(hd, qd), w1=(f, hd), w3=(f, hd), w2=(hd, f)).items():
        w[name] = (rng.integers(0, 256, size=(n, rb(k)), dtype=np.uint8), n, k)
    head = rng.integers(0, 256, size=(head_rows, hd // 32 * 34), dtype=np.uint8)
    per_block = 2 * BLOCK * kvd
    nb = (L + BLOCK - 1) // BLOCK
    pool = rng.integers(0, 0x3C00, size=nb * per_block, dtype=np.uint16)
    bt = list(range(nb))
    x = rng.standard_normal((1, hd)).astype(np.float32)
    ones = np.ones(hd, dtype=np.float32)
    scale = np.float32(1.0 / math.sqrt(c["head_dim"]))
    ex = ThreadPoolExecutor(max_workers=threads) if threads > 1 else None

    def rows_parallel(fn, a, wbytes, n, k):
        """fn(a, weight rows, 1, rows, k) on `threads` slices of the rows (the C code runs without the GIL)"""
        if ex is None:
            return fn(a, wbytes, 1, n, k)
        cuts = [n * i // threads for i in range(threads + 1)]
        parts = list(ex.map(lambda i: fn(a, wbytes[cuts[i]:cuts[i + 1]], 1, cuts[i + 1] - cuts[i], k), range(threads)))
        return np.concatenate(parts, axis=1)

    mm = lambda a, name: rows_parallel(nx.matmul_q4_0, a, w[name][0], w[name][1], w[name][2])
    t0 = time.perf_counter()
    for _ in range(sample_layers):
        nrm = nx.rmsnorm(x, ones, 1, hd, 1e-5)
        q, k, v = mm(nrm, "wq"), mm(nrm, "wk"), mm(nrm, "wv")
        q, k = nx.rope(q, k, c["head_dim"], c["num_heads"], c["num_kv_heads"], 1, L - 1, 0, 10000.0, False)
        nx.reshape_paged_kv(k, pool, [bt[(L - 1) // BLOCK]], [(L - 1) % BLOCK], c["num_kv_heads"], c["head_dim"], BLOCK, False)
        nx.reshape_paged_kv(v, pool, [bt[(L - 1) // BLOCK]], [(L - 1) % BLOCK], c["num_kv_heads"], c["head_dim"], BLOCK, True)
        a = nx.sdpa_paged_decode(q, pool, bt, nb, BLOCK, c["num_heads"], c["num_kv_heads"], c["head_dim"], scale,
                                 L - (nb - 1) * BLOCK).reshape(1, -1)
        x = nx.add(x, mm(a, "wo"))
        nrm = nx.rmsnorm(x, ones, 1, hd, 1e-5)
        g, u = mm(nrm, "w1"), mm(nrm, "w3")
        x = nx.add(x, mm(nx.silu_mul(g, u), "w2"))
    t_layers = time.perf_counter() - t0
    t0 = time.perf_counter()
    rows_parallel(lambda a_, w_, m_, n_, k_: nx.matmul_quant(nx.FMT_Q8_0, a_, w_, m_, n_, k_),
                  nx.rmsnorm(x, ones, 1, hd, 1e-5), head, head_rows, hd)
    t_head = time.perf_counter() - t0
    if ex is not None:
        ex.shutdown()
    per_token = t_layers / sample_layers * c["num_layers"] + t_head / head_rows * c["vocab"]
    what = "%d of %d layers + %d of %d lm_head rows for one sequence (ctx %d), extrapolated to a full token; random " \
           "bytes stand for the weights (values differ from the GPU run's, the time does not depend on them); " \
           % (sample_layers, c["num_layers"], head_rows, c["vocab"], L)
    if threads == 1:
        what += "host has %d cores, the reference path uses min(cores, M)=1" % os.cpu_count()
    else:
        what += "NOT reference behaviour: each matmul's weight rows cut into %d slices run side by side " \
                "(attention and the element-wise steps on one core)" % threads
    return dict(value=1.0 / per_token, unit="tok/s", cores=threads, kind="port", sample=what)


def time_step_gemms(be, mr, c, rows):
    """The decode step's four projection launches per layer (Q|K|V, Wo, gate|up, down) at `rows` activation rows,
    timed with HIP events on the backend's stream over the model's own weights: every layer's matrices once per
    pass, so each launch streams its weights from HBM as in the step. Algorithmic bytes per launch:
    N*K*bytes_per_element + rows*K*4 + rows*N*4. -> dict for the bench line."""
    bpe = {1: 18 / 32, 2: 34 / 32, 3: 144 / 256, 4: 210 / 256}
    lw = mr.layer_weights
    h, f = c["hidden"], c["ffn"]
    rng = np.random.default_rng(9)
    acts = {k: be.upload(rng.standard_normal((rows, k)).astype(np.float32), permanent=True) for k in {h, f, lw[0]["wo"][3]}}

    def group(names):
        """(fmt, pointer, total rows, k) of matrices laid out back to back, else None"""
        ws = [lw[0][n] for n in names]
        fmt, k = ws[0][0], ws[0][3]
        per_layer = []
        for l in lw:
            p, n = l[names[0]][1], 0
            for nm in names:
                if l[nm][1] != p + int(n * k * bpe[fmt]) or l[nm][0] != fmt or l[nm][3] != k:
                    return None
                n += l[nm][2]
            per_layer.append(p)
        return fmt, per_layer, n, k

    shapes = [("Q|K|V", group(["wq", "wk", "wv"])), ("Wo", group(["wo"])), ("gate|up", group(["w1", "w3"])),
              ("down", group(["w2"]))]
    if any(g is None for _, g in shapes):
        for p in acts.values():
            be.free(p)
        return None
    nmax = max(g[2] for _, g in shapes)
    out = be.alloc_permanent(rows * nmax * 4)
    res, total_us, total_bytes = {}, 0.0, 0
    for name, (fmt, ptrs, n, k) in shapes:
        be.prepare_act(acts[k], rows, k)
        reps = 3
        timed = []
        for dst in (None, out):       # the launch alone, as the step issues it; then with its reduction kernel
            for p in ptrs[:2]:
                be.matmul_quant_prepared(fmt, p, dst, None, rows, n, k)
            be.sync()
            be.timer_start()
            for _ in range(reps):
                for p in ptrs:
                    be.matmul_quant_prepared(fmt, p, dst, None, rows, n, k)
            timed.append(be.timer_stop_ms() * 1e3 / (reps * len(ptrs)))
        kernel = be.last_matmul_kernel()
        us = timed[0]
        nbytes = int(n * k * bpe[fmt]) + rows * k * 4 + rows * n * 4
        res[name] = {"n": n, "k": k, "us": round(us, 2), "us_with_reduction": round(timed[1], 2), "bytes": nbytes,
                     "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4), "kernel": kernel}
        if name == "Q|K|V":
            fused = time_fused_qkv(be, lw, c, rows, acts[k])
            if fused is not None:   # what the step launches for Q|K|V: the projection with RoPE and the KV store in its epilogue
                res[name]["us_projection_alone"] = res[name]["us"]
                res[name]["kernel_projection_alone"] = res[name]["kernel"]
                res[name]["kernel"] = be.last_matmul_kernel()
                res[name]["us"] = us = round(fused, 2)
                res[name]["frac"] = round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)
        total_us += us
        total_bytes += nbytes
    be.free(out)
    for p in acts.values():
        be.free(p)
    return {"bound": "hbm", "kernel": "%s (the step's four projection launches per layer, M=%d)"
                                      % (" / ".join(sorted({v["kernel"] for v in res.values()})), rows),
            "achieved": total_bytes / total_us / 1e3, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": total_bytes / total_us / 1e3 / HBM_PEAK_GBS,
            "traffic": GEMM_TRAFFIC_PER_ALGORITHMIC_BYTE * total_bytes if rows == BATCH else None,
            "bytes_per_layer": total_bytes,
            "us_per_layer": total_us, "launches": res,
            "note": "HIP events around back-to-back launches over all layers' weights; us: the projection launch alone, "
                    "as the fused decode blocks issue it (K slices' sums consumed by the next prepare kernel; Q|K|V: "
                    "with its RoPE + KV-store epilogue, timed as vx_decode_attn_qkv minus the prepare kernel alone); "
                    "us_with_reduction: with the separate reduction kernel of the unfused call"}


def time_fused_qkv(be, lw, c, rows, x):
    """The decode step's Q|K|V launch by itself: vx_decode_attn_qkv (RMSNorm prepare, then the projection that rotates
    Q and K from the step's table of angles and stores K and V into a paged pool) over every layer's weights, minus
    the prepare kernel timed alone. A scratch pool of 2 * rows slots takes the stores. None when the fused entry point
    does not take these weights."""
    from vexel_amd import lib
    hq, hk, d, h = c["num_heads"], c["num_kv_heads"], c["head_dim"], c["hidden"]
    qws = [[be.qweight(*l[n]) for n in ("wq", "wk", "wv")] for l in lw]
    if rows > 32 or not be.decode_attn_qkv_supported(*qws[0], d):
        return None
    kvd = hk * d
    nblocks = (2 * rows + BLOCK - 1) // BLOCK
    pool = be.alloc_permanent(nblocks * 2 * BLOCK * kvd * 2)
    dq = be.alloc_permanent(rows * hq * d * 4)
    ones = be.upload(np.ones(h, dtype=np.float32), permanent=True)
    dpos = be.upload(np.arange(100, 100 + rows, dtype=np.int32), permanent=True)
    dslots = be.upload(np.arange(rows, dtype=np.int32), permanent=True)
    theta = float(c.get("rope_theta", 10000.0))
    reps = 3

    def fused(q):
        be.decode_attn_qkv(x, ones, 1e-5, False, q[0], q[1], q[2], rows, dpos, dslots, pool, True, hq, hk, d, BLOCK, theta, dq)

    be.rope_table_prepare(dpos, rows, d, theta)
    for q in qws[:2]:
        fused(q)
    be.sync()
    be.timer_start()
    for _ in range(reps):
        for q in qws:
            fused(q)
    both = be.timer_stop_ms() * 1e3 / (reps * len(qws))
    be.timer_start()
    for _ in range(reps * len(qws)):
        be.rmsnorm_prepare(x, ones, None, rows, h, 1e-5)
    prep = be.timer_stop_ms() * 1e3 / (reps * len(qws))
    for p in (pool, dq, ones, dpos, dslots):
        be.free(p)
    return both - prep


def kernel_report(be):
    """Per-kernel timings through the C ABI, inputs resident in HBM, HIP events on the backend stream. Every
    weight shape cycles over enough distinct copies (> 400 MB) that nothing is served from the 256 MB
    memory-side cache. Algorithmic bytes of a quantized matmul: N*K*bytes_per_element + M*K*4 + M*N*4 with the GGUF
    bytes per element. The matrices are packed at load time as the host runtime packs a batched model's (formats
    with a packed form; one row reads the GGUF rows either way); several rows are timed as the unfused call: the
    projection launch and the reduction of its K slices."""
    synth = load_synth()
    bpe = {1: 18 / 32, 2: 34 / 32, 3: 144 / 256, 4: 210 / 256, 5: 22 / 32, 6: 176 / 256}
    names = {1: "Q4_0", 2: "Q8_0", 3: "Q4_K", 4: "Q6_K", 5: "Q5_0", 6: "Q5_K"}
    shapes = [("Q|K|V", 12288, 4096), ("Wo", 4096, 4096), ("gate|up", 22016, 4096), ("down", 4096, 11008),
              ("lm_head", 32000, 4096)]
    a = np.random.default_rng(0).standard_normal((256, 11008)).astype(np.float32)
    da = be.upload(a, permanent=True)
    print("%-8s %-5s %3s %6s %6s %9s %9s %7s" % ("matmul", "fmt", "M", "N", "K", "us/call", "GB/s", "of 8TB"))
    for fmt in (1, 2, 3, 4, 5, 6):
        for name, n, k in shapes:
            rb = int(k * bpe[fmt])
            copies = max(2, int(400e6 // (n * rb)) + 1)
            ws = []
            for i in range(copies):
                p = be.alloc_permanent(n * rb)
                if fmt >= 5:   # random codes from the host; the f16 scale fields set to small finite values
                    blk = 22 if fmt == 5 else 176
                    raw = np.random.default_rng(77 + i).integers(0, 256, (n * rb // blk, blk), dtype=np.uint8)
                    raw[:, 0:2] = np.frombuffer(np.float16(0.01).tobytes(), dtype=np.uint8)
                    if fmt == 6:
                        raw[:, 2:4] = np.frombuffer(np.float16(0.005).tobytes(), dtype=np.uint8)
                    be.to_device(p, raw)
                    rc = 0
                elif fmt <= 2:
                    rc = synth.vxs_gaussian_quant(fmt, p, n * (k // 32), 0.02, 77 + i)
                else:   # timing does not depend on the codes
                    rc = synth.vxs_random_kquant(fmt, p, n * (k // 256), 77 + i)
                if rc:
                    raise RuntimeError("synthetic weight generation failed: %d" % rc)
                be.qweight_pack(be.qweight(fmt, p, n, k))
                ws.append(p)
            for m in (1, 32, 64, 256):
                out = be.alloc_permanent(m * n * 4)
                be.prepare_act(da, m, k)
                for w in ws[:2]:
                    if m == 1:
                        be.matmul_quant(fmt, da, w, out, None, m, n, k)
                    else:
                        be.matmul_quant_prepared(fmt, w, out, None, m, n, k)
                be.sync()
                reps = 3
                be.timer_start()
                for _ in range(reps):
                    for w in ws:
                        if m == 1:   # the matrix-vector kernel reads the float32 activation itself
                            be.matmul_quant(fmt, da, w, out, None, m, n, k)
                        else:
                            be.matmul_quant_prepared(fmt, w, out, None, m, n, k)
                us = be.timer_stop_ms() * 1e3 / (reps * copies)
                nbytes = n * rb + m * k * 4 + m * n * 4
                gbs = nbytes / us / 1e3
                print("%-8s %-5s %3d %6d %6d %9.1f %9.0f %7.3f" % (name, names[fmt], m, n, k, us, gbs, gbs / HBM_PEAK_GBS))
                be.free(out)
            for w in ws:
                be.free(w)
    be.free(da)
    # attention at the north-star contexts
    ctx = ragged_contexts()
    c = dict(CFG)
    mr, ids = build_model(be, ctx, 8, 4)
    # one decode step, so that the attention call below is the step's own (metadata from the packing kernel)
    first = np.random.default_rng(3).integers(0, c["vocab"], len(ctx)).astype(np.int32)
    mr.decode_graph(first, ids, ctx, 1, use_graph=False)
    ctx = [L + 1 for L in ctx]
    ms = time_attention_kernel(be, mr, ctx, c, 4, reps=40, from_step=True)
    nb = attention_bytes(ctx, c)
    print("paged decode attention, 32 ragged sequences (sum ctx %d), one layer: %.1f us, %.0f GB/s, %.3f of 8 TB/s"
          % (sum(ctx), ms * 1e3, nb / ms / 1e6, nb / ms / 1e6 / HBM_PEAK_GBS))
    mr.close()
    # grouped-query geometries (the matrix-core form of the kernel) as a decode step launches them: a model of that
    # head geometry (small FFN and vocabulary) takes one step, whose packing kernel leaves the attention work list;
    # the launches cycle over enough layers' pools (> 450 MB) that none is served from the memory-side cache
    for hq, hk, nseq, med in ((32, 8, 64, 512), (32, 8, 32, 1024), (28, 4, 32, 1024)):
        rng = np.random.default_rng(0)
        d = 128
        gctx = [int(x) for x in np.clip(np.exp(rng.normal(math.log(med), 0.6, nseq)), 16, 4096)]
        kv_bytes = sum(2 * L * hk * d * 2 for L in gctx)
        layers = -(-450_000_000 // kv_bytes)
        gc = dict(num_layers=layers, hidden=hq * d, num_heads=hq, num_kv_heads=hk, head_dim=d, ffn=1024, vocab=1024)
        mr, ids = build_model(be, gctx, 8, layers, cfg=gc)
        first = np.random.default_rng(3).integers(0, gc["vocab"], nseq).astype(np.int32)
        mr.decode_graph(first, ids, gctx, 1, use_graph=False)
        gctx = [L + 1 for L in gctx]
        ms = time_attention_kernel(be, mr, gctx, gc, layers, reps=10 * layers, from_step=True)
        nb = attention_bytes(gctx, gc)
        print("paged decode attention, %d / %d heads x %d, %d ragged sequences (sum ctx %d), one layer: %.1f us, %.0f GB/s, "
              "%.3f of 8 TB/s" % (hq, hk, d, nseq, sum(gctx), ms * 1e3, nb / ms / 1e6, nb / ms / 1e6 / HBM_PEAK_GBS))
        mr.close()
    # dense causal prefill attention of one 512-token chunk, 7B head geometry (f16 matrix cores, operands as hi + lo halves)
    S, hq, d = 512, c["num_heads"], c["head_dim"]
    rng = np.random.default_rng(5)
    dq = be.upload(rng.standard_normal((S, hq * d)).astype(np.float32), permanent=True)
    dk = be.upload(rng.standard_normal((S, hq * d)).astype(np.float32), permanent=True)
    dv = be.upload(rng.standard_normal((S, hq * d)).astype(np.float32), permanent=True)
    do = be.alloc_permanent(S * hq * d * 4)
    scale = 1.0 / math.sqrt(d)
    for _ in range(3):
        be.sdpa_prefill(dq, dk, dv, do, S, hq, hq, d, scale)
    be.sync()
    be.timer_start()
    for _ in range(20):
        be.sdpa_prefill(dq, dk, dv, do, S, hq, hq, d, scale)
    ms = be.timer_stop_ms() / 20
    flops = 4.0 * hq * d * S * (S + 1) / 2
    print("causal prefill attention, S=512, %d heads x %d: %.1f us, %.1f TFLOP/s algorithmic (x3 on the matrix cores: "
          "hi*hi + hi*lo + lo*hi), %.3f of the 2500 TFLOP/s f16 MFMA peak"
          % (hq, d, ms * 1e3, flops / ms / 1e9, 3 * flops / ms / 1e9 / 2500.0))
    for p_ in (dq, dk, dv, do):
        be.free(p_)


def counter_probe(be, mr, ctx, c, layers):
    """Workload for hardware-counter runs: plain_copy_kernel moves 1 GiB (known traffic, the scale for
    FETCH_SIZE / WRITE_SIZE), then the attention kernel runs 8 times on the benchmark contexts, then the step's
    four quantized projection launches per layer run over every layer's weights."""
    synth = load_synth()
    n = 1 << 30
    src, dst = be.alloc_permanent(n), be.alloc_permanent(n)
    rc = synth.vxs_plain_copy(C.c_void_p(dst), C.c_void_p(src), C.c_int64(n))
    if rc:
        raise RuntimeError("plain copy failed: %d" % rc)
    ms = time_attention_kernel(be, mr, ctx, c, layers, reps=8)
    gm = time_step_gemms(be, mr, c, len(ctx))   # every layer's four projection launches, weights streamed from HBM
    print(json.dumps({"probe": "plain_copy_kernel 1 GiB + 8 attention launches + the step's projection launches",
                      "attention_bytes": attention_bytes(ctx, c), "attention_ms": ms,
                      "projection_launches": gm["launches"] if gm else None}))


def prefill_probe(be, rows=512, reps=10):
    """Workload for MFMA counters (rocprofv3 --pmc SQ_INSTS_VALU_MFMA_MOPS_F16 ...): the four 7B-shaped Q4_0
    projections with `rows` activation rows through the batched MFMA kernel, and one causal prefill attention of
    `rows` tokens (32 heads x 128), `reps` launches each; prints flops and event-timed durations."""
    synth = load_synth()
    shapes = [("Q|K|V", 12288, 4096), ("Wo", 4096, 4096), ("gate|up", 22016, 4096), ("down", 4096, 11008)]
    a = np.random.default_rng(0).standard_normal((rows, 11008)).astype(np.float32)
    da = be.upload(a, permanent=True)
    out = {"rows": rows, "gemm": [], "note": "the GEMM's MFMA work is twice 2*M*N*K: activations enter as hi + lo f16"}
    for name, n, k in shapes:
        rb = k // 32 * 18
        w = be.alloc_permanent(n * rb)
        if synth.vxs_gaussian_quant(1, w, n * (k // 32), 0.02, 91):
            raise RuntimeError("synthetic weight generation failed")
        o = be.alloc_permanent(rows * n * 4)
        be.qweight_pack(be.qweight(1, w, n, k))      # as the host runtime does at load time
        be.prepare_act(da, rows, k)
        be.matmul_quant_prepared(1, w, o, None, rows, n, k)
        be.sync()
        be.timer_start()
        for _ in range(reps):
            be.matmul_quant_prepared(1, w, o, None, rows, n, k)
        ms = be.timer_stop_ms() / reps
        flops = 2.0 * rows * n * k
        out["gemm"].append({"name": name, "n": n, "k": k, "ms": ms, "algorithmic_tflops": flops / ms / 1e9,
                            "mfma_tflops": 2 * flops / ms / 1e9})
        be.free(w)
        be.free(o)
    hq, d = CFG["num_heads"], CFG["head_dim"]
    rng = np.random.default_rng(5)
    bufs = [be.upload(rng.standard_normal((rows, hq * d)).astype(np.float32), permanent=True) for _ in range(3)]
    do = be.alloc_permanent(rows * hq * d * 4)
    scale = 1.0 / math.sqrt(d)
    be.sdpa_prefill(bufs[0], bufs[1], bufs[2], do, rows, hq, hq, d, scale)
    be.sync()
    be.timer_start()
    for _ in range(reps):
        be.sdpa_prefill(bufs[0], bufs[1], bufs[2], do, rows, hq, hq, d, scale)
    ms = be.timer_stop_ms() / reps
    flops = 4.0 * hq * d * rows * (rows + 1) / 2
    out["prefill_attention"] = {"tokens": rows, "ms": ms, "tflops": flops / ms / 1e9}
    # a later chunk of a prompt: `rows` query rows at position 3584 over the paged f16 pool, 8B head geometry (32 / 8)
    hk, start = 8, 3584
    nb = (start + rows + BLOCK - 1) // BLOCK
    pool = be.alloc_permanent(nb * 2 * BLOCK * hk * d * 2)
    if synth.vxs_gaussian_f16(pool, nb * 2 * BLOCK * hk * d, 1.0, 7):
        raise RuntimeError("synthetic KV generation failed")
    dbt = be.upload(rng.permutation(nb).astype(np.int32), permanent=True)
    kvl = np.arange(start + 1, start + rows + 1, dtype=np.int32)
    dk = be.upload(kvl, permanent=True)
    args = (bufs[0], pool, dbt, do, dk, nb, BLOCK, hq, hk, d, scale, rows)
    be.sdpa_paged_decode_multiquery(*args, pool_is_f16=True)
    be.sync()
    be.timer_start()
    for _ in range(reps):
        be.sdpa_paged_decode_multiquery(*args, pool_is_f16=True)
    ms = be.timer_stop_ms() / reps
    flops = 4.0 * hq * d * float(kvl.sum())
    out["paged_multiquery_attention"] = {"rows": rows, "position": start, "heads": "%d/%d x %d" % (hq, hk, d), "ms": ms,
                                         "tflops": flops / ms / 1e9}
    print(json.dumps(out))


def configs_report(be, only=None, use_graph=True):
    """Throughput of the benchmark configs other than the north star, each at its real shape (synthetic weights and
    contexts, greedy decode replayed from a hipGraph; config 4 as its two ingredients; config 5 as one verification
    step). Informational: the benchmark line is the north-star workload.
    only: "1" .. "5" runs that config alone ("4": its decode part; "4p": decode and the prefill chunks).
    use_graph=False (--no-graph) issues the same device-driven steps launch by launch (for kernel traces)."""
    from vexel_amd import lib
    from oracle import host_logic as hl
    tiny = dict(num_layers=22, hidden=2048, num_heads=32, num_kv_heads=4, head_dim=64, ffn=5632, vocab=32000)
    l8b = dict(num_layers=32, hidden=4096, num_heads=32, num_kv_heads=8, head_dim=128, ffn=14336, vocab=128256,
               rope_theta=500000.0)
    q4km = {"*": lib.VX_Q4_K, "wv": lib.VX_Q6_K, "w2": lib.VX_Q6_K, "head": lib.VX_Q6_K}

    def decode_rate(name, cfg, fmts, ctx, steps, spare_tokens=0):
        mr, ids = build_model(be, ctx, steps + 16, cfg["num_layers"], cfg, fmts, spare_tokens=spare_tokens)
        first = np.random.default_rng(3).integers(0, cfg["vocab"], len(ctx)).astype(np.int32)
        mr.decode_graph(first, ids, ctx, 4, use_graph=use_graph)
        be.sync()
        t0 = time.perf_counter()
        mr.decode_graph(None, None, None, steps, use_graph=use_graph, batch=len(ctx))
        be.sync()
        dt = time.perf_counter() - t0
        print("%-64s %8.1f tok/s  %7.3f ms/step" % (name, len(ctx) * steps / dt, dt * 1e3 / steps), flush=True)
        return mr, ids

    rng = np.random.default_rng(0)
    want = lambda n: only is None or only[0] == n
    if want("1"):
        mr, _ = decode_rate("config 1: TinyLlama-shaped Q4_0, 1 sequence, ctx 32 + 64 steps", tiny, None, [32], 64)
        mr.close()
    ctx2 = [int(x) for x in rng.integers(128, 2049, 8)]   # (the contexts are drawn whether or not the config runs: same numbers either way)
    if want("2"):
        mr, _ = decode_rate("config 2: TinyLlama-shaped Q4_0, 8 ragged sequences (sum ctx %d)" % sum(ctx2), tiny, None, ctx2, 128)
        mr.close()
    ctx3 = ragged_contexts()
    if want("3"):
        mr, _ = decode_rate("config 3: 7B-shaped Q4_K_M mix, 32 ragged sequences (sum ctx %d)" % sum(ctx3), CFG, q4km, ctx3, 64)
        mr.close()
    ctx4 = [int(x) for x in np.clip(np.exp(rng.normal(math.log(512.0), 0.6, 64)), 16, 4096)]
    if want("4"):
        _config4(be, rng, ctx4, l8b, decode_rate, prefill=only != "4")
    else:
        rng.integers(0, l8b["vocab"], 512)
    if want("5"):
        _config5(be, rng)


def _config4(be, rng, ctx4, l8b, decode_rate, prefill):
    from vexel_amd import lib
    mr, ids = decode_rate("config 4 (decode part): 8B-shaped Q8_0, 64 sequences (sum ctx %d)" % sum(ctx4), l8b,
                          {"*": lib.VX_Q8_0}, ctx4, 32, spare_tokens=4200)   # (free blocks for the chunks below)
    chunk = rng.integers(0, l8b["vocab"], 512).tolist()
    if not prefill:
        mr.close()
        return
    mr.prefill_with_paged_kv(chunk, 1000, 0)                # (untimed: sizes the workspaces for 512 rows)
    mr.delete_sequence(1000)
    be.sync()
    t0 = time.perf_counter()
    mr.prefill_with_paged_kv(chunk, 1001, 0)
    be.sync()
    dt = time.perf_counter() - t0
    print("%-64s %8.1f tok/s  %7.3f ms/chunk" % ("config 4 (prefill part): one 512-token chunk", 512 / dt, dt * 1e3), flush=True)
    # later chunks of a long prompt: 512 tokens at start positions 512 and 3584 (paged multi-query attention over the
    # f16 pool, runtime/block.go:881-890); the contexts before them are adopted blocks of the synthetic pool
    mr.delete_sequence(1001)
    for start in (512, 3584):
        sid = 2000 + start
        free_now = mr.block_stats()[1] // l8b["num_layers"]
        need = (start + 512 + BLOCK - 1) // BLOCK
        if free_now < need + 2:
            print("config 4 later chunk at %d: skipped, %d free blocks" % (start, free_now), flush=True)
            continue
        mr.create_sequence(sid)
        for p0 in range(0, start, 512):          # the earlier chunks, untimed
            mr.prefill_with_paged_kv(chunk, sid, p0)
        be.sync()
        t0 = time.perf_counter()
        mr.prefill_with_paged_kv(chunk, sid, start)
        be.sync()
        dt = time.perf_counter() - t0
        print("%-64s %8.1f tok/s  %7.3f ms/chunk" % ("config 4 (prefill part): 512-token chunk at position %d" % start,
                                                      512 / dt, dt * 1e3), flush=True)
        mr.delete_sequence(sid)
    mr.close()


def _config5(be, rng):
    from vexel_amd import lib
    from oracle import host_logic as hl
    ctx5 = [int(x) for x in rng.integers(256, 2049, 16)]
    mr, ids = build_model(be, ctx5, 64, 32, CFG, {"*": lib.VX_Q6_K}, max_batch=16)
    start, inputs = list(ctx5), rng.integers(0, 32000, 16).tolist()
    for it in range(4):
        trees = []
        for _ in range(16):
            toks = [rng.choice(32000, 2, replace=False).tolist() for _ in range(4)]
            trees.append(hl.build_candidate_tree_from_topk(toks, [[2.0, 1.0]] * 4, 15).linearize())
        be.sync()
        t0 = time.perf_counter()
        acc, fin, _ = mr.verify_tree(ids, inputs, start, trees, want_logits=False)
        dt = time.perf_counter() - t0
        start = [start[i] + 1 + len(acc[i]) for i in range(16)]
        inputs = fin
    print("%-64s %8.1f rows/s %7.3f ms/step" % ("config 5: 7B-shaped Q6_K, 16 sequences (sum ctx %d), 15-node trees" % sum(ctx5),
                                                  256 / dt, dt * 1e3), flush=True)
    mr.close()


def medusa_report(be):
    """Medusa head inference (medusa/heads.go:83-171) at the 7B shape: all heads' FC1 / FC2 in one pass, then the
    per-head top-k. Weights are float32; GB/s counts the weight bytes against the 8 TB/s HBM peak."""
    rng = np.random.default_rng(0)
    print("heads hidden  vocab rows  forward ms  GB/s  of 8TB  top-10 ms")
    for heads, h, v, rows in ((4, 4096, 32000, 1), (4, 4096, 32000, 8), (4, 2048, 32000, 1), (4, 4096, 128256, 1)):
        d1 = be.alloc_permanent(heads * h * h * 4)
        d2 = be.alloc_permanent(heads * h * v * 4)
        piece = (rng.standard_normal(h * 1000) * 0.02).astype(np.float32)
        for base, total in ((d1, heads * h * h), (d2, heads * h * v)):
            off = 0
            while off < total:
                n = min(piece.size, total - off)
                be.to_device(base + off * 4, piece[:n])
                off += n
        dh = be.upload(rng.standard_normal((rows, h)).astype(np.float32), permanent=True)
        di, dl = be.alloc_permanent(heads * rows * h * 4), be.alloc_permanent(heads * rows * v * 4)
        dk, dv = be.alloc_permanent(heads * rows * 10 * 4), be.alloc_permanent(heads * rows * 10 * 4)
        for _ in range(3):
            be.medusa_forward(dh, d1, d2, di, dl, rows, heads, h, v)
        be.sync()
        be.timer_start()
        for _ in range(20):
            be.medusa_forward(dh, d1, d2, di, dl, rows, heads, h, v)
        ms = be.timer_stop_ms() / 20
        be.timer_start()
        for _ in range(20):
            be.topk_rows(dl, heads * rows, v, 10, dk, dv)
        ms_k = be.timer_stop_ms() / 20
        gbs = heads * (h * h + h * v) * 4 / ms / 1e6
        print("%5d %6d %6d %4d  %10.3f %5.0f  %6.3f  %9.3f" % (heads, h, v, rows, ms, gbs, gbs / 8000, ms_k), flush=True)
        for ptr in (d1, d2, dh, di, dl, dk, dv):
            be.free(ptr)


def arch_report(be):
    """Batched greedy decode (32 ragged sequences, device-driven hipGraph loop) for the layer graphs beside LLaMA at
    the shapes of published models, Q4_0 weights: Qwen 2 7B (fused decode blocks with the bias / split-pair epilogue),
    Phi-2 and Gemma 2 2B (one call per operation)."""
    from vexel_amd import lib
    models = [
        ("LLaMA-2 7B", dict(hidden=4096, num_heads=32, num_kv_heads=32, head_dim=128, ffn=11008, vocab=32000, eps=1e-5,
                            rope_theta=10000.0), 32, None),
        ("Qwen 2 7B", dict(hidden=3584, num_heads=28, num_kv_heads=4, head_dim=128, ffn=18944, vocab=152064, eps=1e-6,
                           rope_theta=1000000.0), 28, dict(rope_neox=True, bias="qkv")),
        ("Phi-2 2.7B", dict(hidden=2560, num_heads=32, num_kv_heads=32, head_dim=80, ffn=10240, vocab=51200, eps=1e-5,
                            rope_theta=10000.0), 32,
         dict(norm_type="layer", mlp_type="gelu", parallel_residual=True, rope_dim=32, rope_neox=True, bias="all")),
        ("Gemma 2 2B", dict(hidden=2304, num_heads=8, num_kv_heads=4, head_dim=256, ffn=9216, vocab=256000, eps=1e-6,
                            rope_theta=10000.0), 26,
         dict(mlp_type="geglu", post_norms=True, attn_softcap=50.0, final_softcap=30.0, embedding_scale=48.0)),
    ]
    ctx = ragged_contexts()
    print("%-12s %6s %7s %10s %9s" % ("model", "layers", "batch", "ms/step", "tok/s"))
    for name, cfg, layers, arch in models:
        c = dict(CFG)
        c.update(cfg)
        mr, ids = build_model(be, ctx, 48, layers, cfg=c, arch=arch)
        first = np.random.default_rng(3).integers(0, c["vocab"], len(ctx)).astype(np.int32)
        mr.decode_graph(first, ids, list(ctx), 4)
        _, ms = mr.decode_graph(None, None, None, 24, batch=len(ctx))
        print("%-12s %6d %7d %10.3f %9.0f" % (name, layers, len(ctx), ms, len(ctx) / ms * 1e3), flush=True)
        mr.close()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=32)
    ap.add_argument("--warmup", type=int, default=4)
    ap.add_argument("--layers", type=int, default=CFG["num_layers"], help="debug only: fewer layers is NOT the benchmark")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--seqs", type=int, default=BATCH, help="debug only: another batch size is NOT the benchmark "
                                                             "(1 = single-stream decode through the matrix-vector kernel)")
    ap.add_argument("--kernel-report", action="store_true",
                    help="time the path's kernels one by one (quantized GEMM shapes per format, attention) and print a "
                         "table of achieved GB/s against the 8 TB/s HBM peak, then exit")
    ap.add_argument("--counter-probe", action="store_true",
                    help="for rocprofv3 --pmc runs: one 1 GiB plain copy and 8 attention launches, then exit")
    ap.add_argument("--only", default=None, choices=["1", "2", "3", "4", "4p", "5"],
                    help="with --configs-report: that config alone (4: its decode part, 4p: with the prefill chunks)")
    ap.add_argument("--configs-report", action="store_true",
                    help="decode / prefill / verification rates of benchmark configs 1-5 at their real shapes, then exit")
    ap.add_argument("--prefill-probe", action="store_true",
                    help="for rocprofv3 --pmc runs of the MFMA kernels: 512-row GEMMs of the 7B shapes and one "
                         "512-token prefill attention, then exit")
    ap.add_argument("--arch-report", action="store_true",
                    help="batched decode rates of the Qwen 2 / Phi-2 / Gemma 2 layer graphs at published shapes, then exit")
    ap.add_argument("--medusa-report", action="store_true",
                    help="time the Medusa heads' forward pass and top-k at the 7B shape, then exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    from vexel_amd.backend import HipBackend
    be = HipBackend(0)
    if args.kernel_report:
        kernel_report(be)
        return
    if args.prefill_probe:
        prefill_probe(be)
        return
    if args.configs_report:
        configs_report(be, args.only, use_graph=not args.no_graph)
        return
    if args.medusa_report:
        medusa_report(be)
        return
    if args.arch_report:
        arch_report(be)
        return
    ctx = ragged_contexts(n=args.seqs) if args.seqs != BATCH else ragged_contexts()
    nseq = len(ctx)
    c = dict(CFG)
    c["num_layers"] = args.layers
    mr, ids = build_model(be, ctx, args.steps + args.warmup + 8, args.layers)
    if args.counter_probe:
        counter_probe(be, mr, ctx, c, args.layers)
        return
    first = np.random.default_rng(3).integers(0, c["vocab"], nseq).astype(np.int32)
    use_graph = not args.no_graph
    # warmup (untimed): first call runs one eager step, captures the graph, replays the rest
    w = max(args.warmup, 2 if use_graph else 1)
    mr.decode_graph(first, ids, ctx, w, use_graph=use_graph)
    be.sync()
    t0 = time.perf_counter()
    toks, ms_events = mr.decode_graph(None, None, None, args.steps, use_graph=use_graph, batch=nseq)
    be.sync()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    ctx_now = [L + w + args.steps for L in ctx]
    # dominant kernel: ragged paged attention (one launch per layer per step)
    attn_ms = time_attention_kernel(be, mr, ctx_now, c, args.layers, reps=4 * args.layers, from_step=True)
    attn_bytes = attention_bytes(ctx_now, c)
    achieved = attn_bytes / (attn_ms * 1e-3) / 1e9
    out = {
        "metric": "decode tok/s, 7B Q4_0 x32 ragged seqs; % HBM peak in matvec + attn",
        "value": nseq * args.steps / wall,
        "unit": "tok/s",
        "n_gpus": 1, "steps": args.steps, "warmup": w,
        "ms_per_step": ms_per_step,
        "ms_per_step_hip_events": ms_events,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "LLaMA-2-7B-shaped Q4_0 (Q8_0 embedding+head), %d layers, %d ragged paged-KV seqs, "
                               "ctx lognormal(median 1024, sigma 0.6) in [64,4096] seed 0, sum ctx %d, block 16, "
                               "greedy decode, hipGraph=%s; float32 activations enter the batched matmuls as two f16 halves "
                               "(hi + lo, about 22 significant bits) with float32 accumulation, a single row's "
                               "matrix-vector products as 22-bit fixed point" % (args.layers, nseq, sum(ctx_now), use_graph),
                   "global_batch": nseq},
        "roofline": {"bound": "hbm", "kernel": "paged_decode_f16_kernel<128,1,1>",
                     "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "traffic": ATTN_TRAFFIC_PER_ALGORITHMIC_BYTE * attn_bytes, "bytes_per_launch": attn_bytes, "ms_per_launch": attn_ms},
    }
    gm = time_step_gemms(be, mr, c, nseq) if nseq >= 2 else None
    if gm:
        out["roofline_matmul"] = gm
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(be, mr, ctx_now, c)
        out["cpu_baseline_all_cores"] = cpu_baseline(be, mr, ctx_now, c, sample_layers=4, head_rows=8000,
                                                     threads=min(16, os.cpu_count() or 1))
    mr.close()
    be.close()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
