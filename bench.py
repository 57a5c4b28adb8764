#!/usr/bin/env python3
"""Benchmark of the quantized-GGUF matmul path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-sweep] [--no-ffn] [--no-cpu]

Headline workload (the second of the benchmark configurations): Q4_K GEMV, W 5120x5120 (102400 super-blocks, 14745600 B),
x f32[5120], batch 1. One "step" is one GEMV. Steps rotate over 64 distinct copies of the weight
(944 MB, larger than the 256 MB Infinity Cache) so every step streams its weight bytes from HBM;
the same loop over ONE copy is reported as the cache-resident ("warm") figure beside it.
The K steps are recorded into HIP graphs on one stream (as many graphs of K launches as it takes to walk over all copies)
and timed with HIP events on that stream: a batch replays the graphs back to back until at least 1024 launches ran, the
figure is the median per step over 9 batches (so --steps 20 and --steps 4096 give the same number).

Prints ONE JSON line. `value` = algorithmic bytes per step (weights + x + y) * K / elapsed, in GB/s.
Also measured in the same run and carried in the line: the 64-layer decode weight sweep, the Q4_K_M FFN block at
batch 1/4/8, the Q8_0 GEMV (the reference's CPU-runnable case), the prefill dequant-GEMM and the CPU baseline.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E bandwidth
Q8_0, Q4_K, Q6_K = 8, 12, 14
# HBM bytes per launch of the headline kernel from hardware counters: the figure, the commit it was measured on and the
# commands are in this file, written beside the counter summary it was worked out from
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "gemv_q4k_5120x5120_hbm_traffic.json")


def kernel_source_sha():
    """sha256 (first 16 hex digits) of the streaming mat-vec's source: counter summaries carry it, so a summary taken on other
    code than the one that runs can be told."""
    import hashlib
    h = hashlib.sha256()
    for name in ("gemv.hip", "common.hpp", "deq_at.hpp"):
        with open(os.path.join(ROOT, "ferric_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def headline_traffic():
    """The counter summary of the headline kernel; `stale` says that the kernel's source has changed since it was taken."""
    try:
        with open(TRAFFIC_JSON) as f:
            t = json.load(f)
    except (OSError, ValueError):
        return None
    t["stale"] = t.get("kernel_source_sha16") != kernel_source_sha()
    if t["stale"]:
        log("[bench] WARNING: profiles/gemv_q4k_5120x5120_hbm_traffic.json was measured on other kernel source than this tree holds")
    return t


def log(*a):
    print(*a, file=sys.stderr, flush=True)


class Timer:
    """HIP events on the stream the kernels are launched on."""

    def __init__(self, lib, check, stream):
        self.lib, self.check, self.stream = lib, check, stream
        self.e0, self.e1 = C.c_void_p(), C.c_void_p()
        check(lib.fhip_event_create(C.byref(self.e0)))
        check(lib.fhip_event_create(C.byref(self.e1)))

    def time_ms(self, fn):
        self.check(self.lib.fhip_stream_sync(self.stream.handle))
        self.check(self.lib.fhip_event_record(self.e0, self.stream.handle))
        fn()
        self.check(self.lib.fhip_event_record(self.e1, self.stream.handle))
        self.check(self.lib.fhip_event_sync(self.e1))
        self.check(self.lib.fhip_stream_sync(self.stream.handle))
        ms = C.c_float()
        self.check(self.lib.fhip_event_elapsed_ms(self.e0, self.e1, C.byref(ms)))
        return float(ms.value)

    def steady_ms(self, fn, n=5, warm_ms=20.0):
        """Median of n timings of fn, taken after fn has been replayed for at least warm_ms: the first launches after the
        host has been busy (building the next weight) run at a lower clock, some 10 % slower for a 100 us kernel."""
        spent = 0.0
        while spent < warm_ms:
            spent += max(self.time_ms(fn), 1e-3)
        return sorted(self.time_ms(fn) for _ in range(n))[n // 2]


def weight_bytes(ty, rows, cols):
    vals, b = {Q8_0: (32, 34), Q4_K: (256, 144), Q6_K: (256, 210), 2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24),
               13: (256, 176), 20: (32, 18), 23: (256, 136), 39: (32, 17)}[ty]
    return rows * (cols // vals) * b


def replicate(F, lib, check, host_bytes, ncopy):
    """ncopy copies of one weight's bytes in one HBM allocation (copy 0 uploaded, the rest device copies)."""
    n = host_bytes.size
    buf = F.DeviceBuffer(n * ncopy)
    check(lib.fhip_memcpy_h2d(buf.ptr, host_bytes.ctypes.data_as(C.c_void_p), n, None))
    check(lib.fhip_stream_sync(None))
    for i in range(1, ncopy):
        check(lib.fhip_memcpy_d2d(C.c_void_p(buf.ptr.value + i * n), buf.ptr, n, None))
    check(lib.fhip_stream_sync(None))
    return buf


def gemv_graph(F, lib, check, stream, weights, x, y, steps, swiglu=False, first=0):
    g = F.Graph.begin(stream)
    fn = lib.fhip_matmul_q_swiglu if swiglu else lib.fhip_matmul_q
    for i in range(steps):
        check(fn(weights[(first + i) % len(weights)].handle, x.buf.ptr, x.shape[0], y.buf.ptr, stream.handle))
    return g.end()


def time_per_launch(timer, graphs, launches_per_graph, min_launches=1024, batches=9):
    """Median over `batches` batches of the time per launch. A batch replays the graphs round-robin, back to back inside one
    event pair, often enough for at least `min_launches` launches: a single short graph (20 launches are 0.1 ms) would be
    timed with the graph's start-up and the clock ramp in it."""
    reps = max(1, -(-min_launches // (launches_per_graph * len(graphs))))

    def batch():
        for _ in range(reps):
            for g in graphs:
                g.launch()
    batch()
    ts = sorted(timer.time_ms(batch) for _ in range(batches))
    return ts[len(ts) // 2] / (reps * len(graphs) * launches_per_graph)


def rotating_graphs(make, steps, ncopy):
    """Graphs of `steps` launches each that together walk over all `ncopy` weight copies in order, so that replaying them
    round-robin never returns to a copy before every other copy has been read."""
    n = 1 if steps >= ncopy else -(-ncopy // steps)
    return [make(j * steps) for j in range(n)]


def bench_gemv(F, lib, check, stream, timer, ty, rows, cols, steps, warmup, seed, x_seed, ncopy, cold_only=False, with_reader=False, bits=None):
    from ferric_amd.synth import synth_weights
    nbytes = weight_bytes(ty, rows, cols)
    host = synth_weights(ty, rows, cols, seed)
    buf = replicate(F, lib, check, host, ncopy)
    ws = [F.QMatrix.wrap_device(buf, nbytes, ty, rows, cols, offset=i * nbytes) for i in range(ncopy)]
    if bits:                                                   # activation precision of these handles (a new handle has 24 bits)
        for w in ws:
            w.matvec_precision(bits)
    x = F.Tensor.from_vec(np.random.default_rng(x_seed).standard_normal(cols).astype(np.float32), (1, cols))
    y = F.Tensor.empty((1, rows))
    alg = nbytes + 4 * cols + 4 * rows
    out = {}
    gemv_graph(F, lib, check, stream, ws, x, y, max(warmup, 1)).launch()          # the untimed warm-up steps
    for name, wl in ((("cold", ws),) if cold_only else (("cold", ws), ("warm", ws[:1]))):
        graphs = rotating_graphs(lambda first: gemv_graph(F, lib, check, stream, wl, x, y, steps, first=first), steps, len(wl))
        ms = time_per_launch(timer, graphs, steps)
        out[name] = {"ms_per_step": ms, "GBps": alg / (ms * 1e-3) / 1e9}
    if with_reader:
        # the same bytes through a kernel that only reads them, same rotation, same timing: what a perfect reader gets
        sink = F.DeviceBuffer(256)

        def reader_graph(first):
            g = F.Graph.begin(stream)
            for i in range(steps):
                check(lib.fhip_debug_read_probe(C.c_void_p(buf.ptr.value + ((first + i) % ncopy) * nbytes), nbytes, sink.ptr, stream.handle))
            return g.end()
        out["reader_ms"] = time_per_launch(timer, rotating_graphs(reader_graph, steps, ncopy), steps)
    return out, alg, nbytes


def bench_q80_batch(F, lib, check, stream, timer, rows=4096, cols=4096, batch=8, ncopy=32):
    """The 4096 x 4096 Q8_0 weight at a batch of 8 activation rows, cold (32 rotating copies, 571 MB): the one-pass f16 hi/lo
    matmul against the exact-f32 mat-vec kernel, which needs a pass over the weights per two rows."""
    from ferric_amd.synth import synth_weights
    nbytes = weight_bytes(Q8_0, rows, cols)
    buf = replicate(F, lib, check, synth_weights(Q8_0, rows, cols, 0), ncopy)
    ws = [F.QMatrix.wrap_device(buf, nbytes, Q8_0, rows, cols, offset=i * nbytes) for i in range(ncopy)]
    x = F.Tensor.from_vec(np.random.default_rng(2).standard_normal((batch, cols)).astype(np.float32), (batch, cols))
    y = F.Tensor.empty((batch, rows))
    scratch = F.DeviceBuffer(max(256, lib.fhip_matmul_q_f16x2_ws_bytes(ws[0].handle, batch)))

    def timed(launch):
        g = F.Graph.begin(stream)
        for w in ws:
            launch(w)
        g.end()
        g.launch()
        return min(timer.time_ms(g.launch) for _ in range(3)) / ncopy * 1e3

    one_pass = timed(lambda w: check(lib.fhip_matmul_q_f16x2(w.handle, x.buf.ptr, batch, y.buf.ptr, scratch.ptr, stream.handle)))
    # the drop-in entry point takes the same kernels for this batch, out of the library's workspace
    check(lib.fhip_workspace_reserve(stream.handle, lib.fhip_workspace_bytes(ws[0].handle, None, batch)))
    drop_in = timed(lambda w: check(lib.fhip_matmul_q(w.handle, x.buf.ptr, batch, y.buf.ptr, stream.handle)))
    for w in ws:
        w.batch_policy(1)                              # FHIP_BATCH_F32_MATVEC
    per_row = timed(lambda w: check(lib.fhip_matmul_q(w.handle, x.buf.ptr, batch, y.buf.ptr, stream.handle)))
    return {"batch": batch, "matmul_q_us": drop_in, "matmul_q_weight_GBps": nbytes / drop_in / 1e3, "f16x2_us": one_pass,
            "f32_matvec_policy_us": per_row}


def launch_floor_us(F, lib, check, stream, timer, n=2048):
    """What one launch costs in a graph on this box when the kernel does nothing to speak of (one workgroup adds 0 to a
    word): the part of every per-launch figure in this file that no kernel can win back."""
    from ferric_amd import decode as X
    w = X._u32_tensor([0])
    g = F.Graph.begin(stream)
    for _ in range(n):
        check(lib.fhip_u32_add(w.buf.ptr, 1, 0, stream.handle))
    g = g.end()
    g.launch()
    check(lib.fhip_stream_sync(stream.handle))
    return min(timer.time_ms(g.launch) for _ in range(3)) * 1e3 / n


def bench_ffn(F, lib, check, stream, timer, batches, reps=20, ncopy=4):
    """The Q4_K_M FFN block (gate|up 2 x (5120 -> 17408) Q4_K, down 17408 -> 5120 Q6_K) on its three paths. Cold figures: the launches of the timed graph rotate over `ncopy`
    distinct copies of both weights (4 x 173 MB = 694 MB > the 256 MB Infinity Cache), so every launch reads HBM; the
    warm figure (one copy, which the cache can hold) is reported beside it for the f32 path."""
    from ferric_amd.synth import synth_weights
    n_embd, n_ff = 5120, 17408
    gbuf = replicate(F, lib, check, synth_weights(Q4_K, 2 * n_ff, n_embd, 3), ncopy)
    dbuf = replicate(F, lib, check, synth_weights(Q6_K, n_embd, n_ff, 4), ncopy)
    gb, db = weight_bytes(Q4_K, 2 * n_ff, n_embd), weight_bytes(Q6_K, n_embd, n_ff)
    gus = [F.QMatrix.wrap_device(gbuf, gb, Q4_K, 2 * n_ff, n_embd, offset=i * gb) for i in range(ncopy)]
    dns = [F.QMatrix.wrap_device(dbuf, db, Q6_K, n_embd, n_ff, offset=i * db) for i in range(ncopy)]
    wbytes = gb + db
    res = {}

    def timed(launch, copies):
        g = F.Graph.begin(stream)
        for i in range(reps):
            launch(gus[i % copies], dns[i % copies])
        g.end()
        g.launch()
        return min(timer.time_ms(g.launch) for _ in range(3)) / reps

    def entry(ms, b):
        return {"ms": ms, "weight_GBps": wbytes / (ms * 1e-3) / 1e9, "tokens_per_s": b / (ms * 1e-3)}

    for b in batches:
        x = F.Tensor.from_vec(np.random.default_rng(5).standard_normal((b, n_embd)).astype(np.float32), (b, n_embd))
        ws, y = F.Tensor.empty((b, n_ff)), F.Tensor.empty((b, n_embd))
        # fhip_ffn, the drop-in entry point: the mat-vec kernels for one and two rows, the one-pass f16 hi/lo kernels from three
        # rows on (out of the library's workspace, reserved here because a capturing stream cannot allocate)
        check(lib.fhip_workspace_reserve(stream.handle, max(lib.fhip_workspace_bytes(gus[0].handle, dns[0].handle, b),
                                                            lib.fhip_workspace_bytes_coop(gus[0].handle, dns[0].handle, b))))
        f32 = lambda gu, dn: check(lib.fhip_ffn(gu.handle, dn.handle, x.buf.ptr, b, y.buf.ptr, ws.buf.ptr, stream.handle))
        res[str(b)] = entry(timed(f32, ncopy), b)
        res[str(b)]["warm_one_copy_ms"] = timed(f32, 1)
        res[str(b)]["path"] = ("streaming mat-vec" if b <= 2 else
                               "gate|up + SwiGLU on the four-row int8 matrix-instruction mat-vec, down on the one-pass f16 hi/lo kernels, cut rows added in a fixed order (FHIP_BATCH_ORDERED)" if b <= 4 else
                               "one-pass f16 hi/lo matrix-core kernels, cut rows added in a fixed order (FHIP_BATCH_ORDERED)")
        if b > 2:
            for policy, key in ((0, "atomic_adds_policy"), (1, "f32_matvec_policy")):   # FHIP_BATCH_AUTO, FHIP_BATCH_F32_MATVEC
                for w in gus + dns:
                    w.batch_policy(policy)
                res[str(b)][key] = entry(timed(f32, ncopy), b)
            for w in gus + dns:
                w.batch_policy(2)
        # the same block through the matrix-core entry point (bf16 operands, f32 accumulate): one pass over
        # the weights for the whole batch
        wsb = F.DeviceBuffer(max(256, lib.fhip_ffn_coop_ws_bytes(gus[0].handle, dns[0].handle, b)))
        coop = lambda gu, dn: check(lib.fhip_ffn_coop(gu.handle, dn.handle, x.buf.ptr, b, y.buf.ptr, wsb.ptr, stream.handle))
        res[str(b)]["matrix_core_path"] = entry(timed(coop, ncopy), b)
        # and through the f16 matrix cores with exact integer weights and hi/lo split activations: one pass over
        # the weights, f32-grade results
        wsh = F.DeviceBuffer(max(256, lib.fhip_ffn_f16x2_ws_bytes(gus[0].handle, dns[0].handle, b)))
        f16 = lambda gu, dn: check(lib.fhip_ffn_f16x2(gu.handle, dn.handle, x.buf.ptr, b, y.buf.ptr, wsh.ptr, stream.handle))
        res[str(b)]["f16x2_path"] = entry(timed(f16, ncopy), b)
    return res, wbytes


def bench_moe(F, lib, check, stream, timer, reps=64):
    """The routed-expert block of a mixture-of-experts decode layer (the callers of the "_id" entry points,
    crates/ferric-llama/src/qwen35.rs:862-871) at Qwen3-30B-A3B's shape: hidden 2048, 128 experts, 8 used, expert FFN
    768; gate|up slab Q4_K [128*1536, 2048] (226 MB), down slab Q6_K [128*2048, 768] (165 MB). One step = router
    top-k on given logits, selected gate|up + SwiGLU, selected down + weighted sum. Each of the `reps` steps in the
    graph uses its own random logits, so different experts are read from step to step (391 MB of slabs)."""
    from ferric_amd.synth import synth_weights
    d, ne, k, eff = 2048, 128, 8, 768
    def slab(ty, rows_pe, cols, seed):   # 8 distinct experts' bytes tiled 16 times: the values do not matter for timing
        one = synth_weights(ty, 8 * rows_pe, cols, seed)
        return F.QMatrix.from_bytes(np.tile(one, ne // 8), ty, ne * rows_pe, cols)
    gu, dn = slab(Q4_K, 2 * eff, d, 60), slab(Q6_K, d, eff, 61)
    res = {}
    for t in (1, 4):
        rng = np.random.default_rng(62 + t)
        x = F.Tensor.from_vec(rng.standard_normal((t, d)).astype(np.float32), (t, d))
        logits = [F.Tensor.from_vec(rng.standard_normal((t, ne)).astype(np.float32) * 2, (t, ne)) for _ in range(reps)]
        selw, mid = F.Tensor.empty((t, 2 * k)), F.Tensor.empty((t, k, eff))
        y, ws = F.Tensor.empty((t, d)), F.Tensor.empty((t * k, d))
        g = F.Graph.begin(stream)
        for i in range(reps):
            check(lib.fhip_moe_topk(logits[i].buf.ptr, None, t, ne, k, 0, 1.0, 1, selw.buf.ptr, stream.handle))
            check(lib.fhip_matmul_q_swiglu_id(gu.handle, x.buf.ptr, t, selw.buf.ptr, k, eff, mid.buf.ptr, stream.handle))
            check(lib.fhip_matmul_q_id_wsum(dn.handle, mid.buf.ptr, t, selw.buf.ptr, k, d, y.buf.ptr, ws.buf.ptr, stream.handle))
        g.end()
        g.launch()
        ms = min(timer.time_ms(g.launch) for _ in range(3)) / reps
        wbytes = t * k * (weight_bytes(Q4_K, 2 * eff, d) + weight_bytes(Q6_K, d, eff))
        res[str(t)] = {"ms": ms, "expert_weight_bytes_read": wbytes, "weight_GBps": wbytes / (ms * 1e-3) / 1e9, "launches": 4}
    return res


def bench_host_entry(F, rows=4096, cols=4096, reps=12):
    """The host-buffer entry points of the CPU path (cpu_simd::matvec_q8_0 and its pooled form): weights, activations and
    results cross PCIe inside the call. Never `value`: it measures the bus, not the kernel."""
    from ferric_amd.synth import synth_weights
    w = synth_weights(Q8_0, rows, cols, 0)
    x = np.random.default_rng(2).standard_normal(cols).astype(np.float32)
    F.matvec_q8_0(x, w, rows, cols)
    t0 = time.perf_counter()
    for _ in range(reps):
        F.matvec_q8_0(x, w, rows, cols)
    each = (time.perf_counter() - t0) / reps
    pool = F.Pool(1)
    F.matvec_q8_0_pooled(pool, x, w, cols, 0, rows)
    t0 = time.perf_counter()
    for _ in range(reps * 4):
        F.matvec_q8_0_pooled(pool, x, w, cols, 0, rows)
    pooled = (time.perf_counter() - t0) / (reps * 4)
    pool.close()
    return {"workload": "Q8_0 4096x4096, host buffers in and out", "matvec_q8_0_host_ms": each * 1e3, "weight_GBps_with_upload": w.size / each / 1e9,
            "matvec_q8_0_pooled_ms": pooled * 1e3, "note": "the pooled call keeps the weight resident and uploads the activations only"}


def bench_gguf(F, lib, check, n_tensors=8, rows=11008, cols=5120):
    """GGUF ingest: a synthetic file of n_tensors Q4_K [rows, cols] tensors (31.7 MB each) written to a temporary
    file, then opened (mmap + header parse + stride check) and every tensor uploaded straight from the mapping.
    Host-side I/O and PCIe: reported for the record, never part of `value`."""
    import struct
    import tempfile
    from ferric_amd.synth import synth_weights
    one = synth_weights(Q4_K, rows, cols, 70).tobytes()
    head = bytearray(b"GGUF" + struct.pack("<IQQ", 3, n_tensors, 0))
    for i in range(n_tensors):
        name = f"blk.{i}.ffn_down.weight".encode()
        head += struct.pack("<Q", len(name)) + name + struct.pack("<IQQIQ", 2, cols, rows, Q4_K, i * len(one))
    head.extend(b"\0" * (-len(head) % 32))
    with tempfile.NamedTemporaryFile(suffix=".gguf") as f:
        f.write(head)
        for _ in range(n_tensors):
            f.write(one)
        f.flush()
        t0 = time.perf_counter()
        g = F.GgufFile.open(f.name)
        t_open = time.perf_counter() - t0
        best = None
        for _ in range(3):
            t0 = time.perf_counter()
            ws = [g.qmatrix(t.name) for t in g.tensors]
            check(lib.fhip_stream_sync(None))
            dt = time.perf_counter() - t0
            best = dt if best is None or dt < best else best
            del ws
        g.close()
    total = n_tensors * len(one)
    return {"file_bytes": total + len(head), "open_parse_ms": t_open * 1e3, "upload_ms": best * 1e3, "upload_GBps": total / best / 1e9,
            "note": "page-cache-resident file, pageable mapping -> hipMemcpy; host I/O and PCIe bound"}


def bench_sweep(F, lib, check, stream, timer, tokens=4, layers=64):
    """The decode weight sweep: per layer fused QKV 5120->7168, O 5120->5120, fused gate+up 5120->34816 (+SwiGLU), all Q4_K,
    down 17408->5120 Q6_K; lm_head 5120->151936 Q6_K. One stream, one graph of layers*4+1 launches. Measured three ways:
    every op on a fixed activation vector with the handles at 16-bit activations (`ms_per_token`, as the headline) and at the
    24 bits a handle has unless told otherwise (`ms_per_token_x24`), and as a true chain in which every op reads what the op before it wrote, held finite by the
    RMS norms fused into the QKV and gate|up mat-vecs (`chained`)."""
    from ferric_amd.synth import synth_weights
    shapes = [("qkv", Q4_K, 7168, 5120), ("o", Q4_K, 5120, 5120), ("gate_up", Q4_K, 34816, 5120), ("down", Q6_K, 5120, 17408)]
    host = {n: synth_weights(ty, r, c, 40 + i) for i, (n, ty, r, c) in enumerate(shapes)}
    layer_bytes = sum(h.size for h in host.values())
    stacks = {n: replicate(F, lib, check, host[n], layers) for n, _, _, _ in shapes}
    head_host = synth_weights(Q6_K, 151936, 5120, 50)
    head_buf, head_bytes = replicate(F, lib, check, head_host, 1), head_host.size
    head = F.QMatrix.wrap_device(head_buf, head_bytes, Q6_K, 151936, 5120)
    total = layer_bytes * layers + head_bytes
    del head_host
    rng = np.random.default_rng(6)
    x = F.Tensor.from_vec(rng.standard_normal(5120).astype(np.float32), (1, 5120))
    h = F.Tensor.from_vec(rng.standard_normal(17408).astype(np.float32) * 0.1, (1, 17408))
    y_qkv, y_o, y_ff, y_dn, logits = (F.Tensor.empty((1, n)) for n in (7168, 5120, 17408, 5120, 151936))
    W = {}
    for n, ty, r, c in shapes:
        nb = host[n].size
        W[n] = [F.QMatrix.wrap_device(stacks[n], nb, ty, r, c, offset=l * nb) for l in range(layers)]
    s = stream.handle

    def timed(record):
        g = F.Graph.begin(stream)
        record()
        g.end()
        g.launch()
        ts = sorted(timer.time_ms(lambda: [g.launch() for _ in range(tokens)]) / tokens for _ in range(5))
        return ts[len(ts) // 2], ts

    def fixed_inputs():
        for l in range(layers):
            check(lib.fhip_matmul_q(W["qkv"][l].handle, x.buf.ptr, 1, y_qkv.buf.ptr, s))
            check(lib.fhip_matmul_q(W["o"][l].handle, x.buf.ptr, 1, y_o.buf.ptr, s))
            check(lib.fhip_matmul_q_swiglu(W["gate_up"][l].handle, x.buf.ptr, 1, y_ff.buf.ptr, s))
            check(lib.fhip_matmul_q(W["down"][l].handle, h.buf.ptr, 1, y_dn.buf.ptr, s))
        check(lib.fhip_matmul_q(head.handle, x.buf.ptr, 1, logits.buf.ptr, s))

    def set_bits(bits):
        for ws in W.values():
            for w in ws:
                w.matvec_precision(bits)
        head.matvec_precision(bits)

    per_bits = {}
    for bits in (24, 16):
        set_bits(bits)
        per_bits[bits] = timed(fixed_inputs)
    ms, ts = per_bits[16]
    # The chain: x -> norm+QKV -> O (on the first 5120 of the QKV row) -> norm+gate|up+SwiGLU -> down -> next layer; the
    # head's norm is a launch of its own (a weight of that size is not fused). 16-bit activations, as ms_per_token.
    norm_w = F.Tensor.from_vec(((rng.random(5120) + 0.5) * 0.01).astype(np.float32), (1, 5120))
    scratch, dn2 = F.Tensor.empty((1, 5120)), [F.Tensor.empty((1, 5120)) for _ in range(2)]

    def chained():
        cur = x
        for l in range(layers):
            check(lib.fhip_norm_matmul_q(W["qkv"][l].handle, cur.buf.ptr, None, norm_w.buf.ptr, 1e-6, None, scratch.buf.ptr, 0, y_qkv.buf.ptr, s))
            check(lib.fhip_matmul_q(W["o"][l].handle, y_qkv.buf.ptr, 1, y_o.buf.ptr, s))
            check(lib.fhip_norm_matmul_q(W["gate_up"][l].handle, y_o.buf.ptr, None, norm_w.buf.ptr, 1e-6, None, scratch.buf.ptr, 1, y_ff.buf.ptr, s))
            check(lib.fhip_matmul_q(W["down"][l].handle, y_ff.buf.ptr, 1, dn2[l % 2].buf.ptr, s))
            cur = dn2[l % 2]
        check(lib.fhip_norm_matmul_q(head.handle, cur.buf.ptr, None, norm_w.buf.ptr, 1e-6, None, scratch.buf.ptr, 0, logits.buf.ptr, s))
    ms_chain, _ = timed(chained)
    finite = bool(np.isfinite(logits.to_vec(stream)).all())
    # The same 257 launches with a kernel that only reads each weight's bytes (fhip_debug_read_probe): what this device gives
    # a sweep cut into these launches when no arithmetic, staging or reduction stands in the way.
    sink = F.DeviceBuffer(256)

    def readers():
        for l in range(layers):
            for n, _, _, _ in shapes:
                check(lib.fhip_debug_read_probe(C.c_void_p(stacks[n].ptr.value + l * host[n].size), host[n].size, sink.ptr, s))
        check(lib.fhip_debug_read_probe(head_buf.ptr, head_bytes, sink.ptr, s))
    floor_ms, _ = timed(readers)
    gbps = lambda t: total / (t * 1e-3) / 1e9
    return {"ms_per_token": ms, "ms_per_token_min_max": [ts[0], ts[-1]], "GBps": gbps(ms), "frac_of_peak": gbps(ms) / HBM_PEAK_GBPS, "activation_bits": 16,
            "ms_per_token_x16": ms,
            "ms_per_token_x24": per_bits[24][0], "GBps_x24": gbps(per_bits[24][0]), "frac_of_peak_x24": gbps(per_bits[24][0]) / HBM_PEAK_GBPS,
            "chained": {"ms_per_token": ms_chain, "GBps": gbps(ms_chain), "launches_per_token": layers * 4 + 2, "logits_finite": finite,
                        "what": "every op reads the op before it: x -> norm+QKV -> O -> norm+gate|up+SwiGLU -> down -> next layer; norm launch + lm_head"},
            "reader_floor_ms": floor_ms, "reader_floor_GBps": gbps(floor_ms), "frac_of_reader": floor_ms / ms,
            "weight_bytes": total, "layers": layers, "launches_per_token": layers * 4 + 1,
            "inputs": "fixed N(0,1) activations per op for ms_per_token (outputs are not fed forward, so values stay finite); "
                      "ops still execute in stream order; `chained` feeds every op the output of the one before"}


def bench_marginal(F, lib, check, stream, timer, sizes=(5120, 20480, 81920, 327680), cols=5120):
    """Time against bytes for Q4_K weights of `cols` columns, one activation row, cold: a least-squares line through the launch
    times of four weight sizes gives what a launch costs whatever its size (`fixed_us`) and the rate at which every further
    byte moves (`marginal_GBps`) -- the reference's own model of a mat-vec call (crates/ferric-tensor/examples/matvec_roofline.rs:37-41).
    The same for the kernel that only reads. Every size rotates over copies that add up to 0.9 GB or more."""
    from ferric_amd.synth import synth_weights
    unit_rows = sizes[0]
    unit = weight_bytes(Q4_K, unit_rows, cols)
    ncopy = max(64, 2 * sizes[-1] // unit_rows)
    buf = replicate(F, lib, check, synth_weights(Q4_K, unit_rows, cols, 1), ncopy)     # big weights are runs of the small one's rows
    x = F.Tensor.from_vec(np.random.default_rng(2).standard_normal(cols).astype(np.float32), (1, cols))
    y = F.Tensor.empty((1, sizes[-1]))
    sink = F.DeviceBuffer(256)
    pts = []
    for rows in sizes:
        per = rows // unit_rows
        n = ncopy // per
        ws = [F.QMatrix.wrap_device(buf, unit * per, Q4_K, rows, cols, offset=i * unit * per) for i in range(n)]
        for w in ws:
            w.matvec_precision(16)                                # as the headline
        launches = max(n, 8)
        g = F.Graph.begin(stream)
        for i in range(launches):
            check(lib.fhip_matmul_q(ws[i % n].handle, x.buf.ptr, 1, y.buf.ptr, stream.handle))
        g = g.end()
        gr = F.Graph.begin(stream)
        for i in range(launches):
            check(lib.fhip_debug_read_probe(C.c_void_p(buf.ptr.value + (i % n) * unit * per), unit * per, sink.ptr, stream.handle))
        gr = gr.end()
        t = time_per_launch(timer, [g], launches, min_launches=max(launches, 256 // per), batches=5) * 1e3
        tr = time_per_launch(timer, [gr], launches, min_launches=max(launches, 256 // per), batches=5) * 1e3
        pts.append({"rows": rows, "bytes": unit * per, "us": t, "reader_us": tr})
        del ws

    def fit(key):
        bx = np.array([p["bytes"] for p in pts], np.float64)
        ty = np.array([p[key] for p in pts], np.float64)
        slope, icept = np.polyfit(bx, ty, 1)                      # us per byte, us
        return {"fixed_us": float(icept), "marginal_GBps": float(1e-3 / slope), "marginal_frac_of_peak": float(1e-3 / slope / HBM_PEAK_GBPS)}
    return {"points": pts, "mat_vec": fit("us"), "reader": fit("reader_us"), "activation_bits": 16,
            "what": f"Q4_K, {cols} columns, batch 1, cold; time = fixed_us + bytes / marginal rate (least squares over the four sizes)"}


def bench_other_shapes(F, lib, check, stream, timer):
    """Cold launch times of the weight shapes of other models that the launch policy was tuned on (besides the benchmark's own):
    a retune that helps one set and hurts the other shows here. `cold_us`: handles at 16-bit activations, as the headline;
    `cold_us_x24`: as the library makes them."""
    from ferric_amd.synth import synth_weights
    shapes = [("q4_k 8192x8192", Q4_K, 8192, 8192, 0), ("q4_k 10240x8192", Q4_K, 10240, 8192, 0), ("q4_k gate|up 57344x8192", Q4_K, 57344, 8192, 1),
              ("q4_k 28672x4096", Q4_K, 28672, 4096, 0), ("q4_k gate|up 22016x4096", Q4_K, 22016, 4096, 1), ("q4_k 4096x4096", Q4_K, 4096, 4096, 0),
              ("q4_k 20480x5120", Q4_K, 20480, 5120, 0), ("q6_k 5120x5120", Q6_K, 5120, 5120, 0), ("q6_k 4096x4096", Q6_K, 4096, 4096, 0),
              ("q6_k 4096x14336", Q6_K, 4096, 14336, 0), ("q6_k 8192x28672", Q6_K, 8192, 28672, 0), ("q6_k 128256x4096", Q6_K, 128256, 4096, 0),
              ("q8_0 12288x4096", Q8_0, 12288, 4096, 0), ("q5_k 5120x5120", 13, 5120, 5120, 0)]
    out = {}
    for name, ty, rows, cols, swiglu in shapes:
        nb = weight_bytes(ty, rows, cols)
        ncopy = max(2, min(48, -(-(600 << 20) // nb)))
        small = synth_weights(ty, min(rows, 2048), cols, 90)       # rows repeat: the values do not matter for timing
        host = np.tile(small, -(-rows // min(rows, 2048)))[:nb]
        buf = replicate(F, lib, check, host, ncopy)
        ws = [F.QMatrix.wrap_device(buf, nb, ty, rows, cols, offset=i * nb) for i in range(ncopy)]
        x = F.Tensor.from_vec(np.random.default_rng(2).standard_normal(cols).astype(np.float32), (1, cols))
        y = F.Tensor.empty((1, rows))
        launches = max(ncopy, 16)
        g = gemv_graph(F, lib, check, stream, ws, x, y, launches, swiglu=bool(swiglu))
        us24 = time_per_launch(timer, [g], launches, min_launches=128, batches=5) * 1e3
        for w in ws:
            w.matvec_precision(16)
        g = gemv_graph(F, lib, check, stream, ws, x, y, launches, swiglu=bool(swiglu))
        us = time_per_launch(timer, [g], launches, min_launches=128, batches=5) * 1e3
        out[name] = {"cold_us": us, "weight_GBps": nb / us / 1e3, "cold_us_x24": us24}
        del ws, buf
    return out


def decode_stack(F, lib, check, layers=64):
    """The 64-layer stack of the decode sweep as a decoder: fused QKV 5120->7168 (40 query / 8 KV heads of 128), O, fused gate|up
    5120->34816, all Q4_K; down 17408->5120 Q6_K; output norm + lm_head 151936 Q6_K. Synthetic weights, one distinct copy per
    layer. Returns (cfg, layers, output norm, lm_head, weight bytes)."""
    from ferric_amd import decode as X
    from ferric_amd.synth import synth_weights
    d, nh, nkv, hd, n_ff, vocab = 5120, 40, 8, 128, 17408, 151936
    shapes = [("qkv", Q4_K, (nh + 2 * nkv) * hd, d), ("o", Q4_K, d, nh * hd), ("gate_up", Q4_K, 2 * n_ff, d), ("down", Q6_K, d, n_ff)]
    host = {n: synth_weights(ty, r, c, 40 + i) for i, (n, ty, r, c) in enumerate(shapes)}
    stacks = {n: replicate(F, lib, check, host[n], layers) for n, _, _, _ in shapes}
    head_host = synth_weights(Q6_K, vocab, d, 50)
    head = F.QMatrix.from_bytes(head_host, Q6_K, vocab, d)
    weight_bytes_total = sum(h.size for h in host.values()) * layers + head_host.size
    del head_host
    rng = np.random.default_rng(8)
    T = lambda a: F.Tensor.from_vec(a, a.shape)
    # block norms small enough that a normalised vector projects to O(1) through the synthetic weights (rows of norm ~ 2 sqrt(cols))
    small, unit = T(((rng.random(d) + 0.5) * 0.01).astype(np.float32)), T((rng.random(hd) + 0.5).astype(np.float32))
    W = {}
    for n, ty, r, c in shapes:
        nb = host[n].size
        W[n] = [F.QMatrix.wrap_device(stacks[n], nb, ty, r, c, offset=l * nb) for l in range(layers)]
    lay = [X.Qwen3Layer(small, W["qkv"][l], W["o"][l], small, W["gate_up"][l], W["down"][l], unit, unit) for l in range(layers)]
    cfg = X.Qwen3Cfg(d, nh, nkv, hd, n_ff, eps=1e-6, rope_base=1e6)
    return cfg, lay, small, head, weight_bytes_total, stacks


def decoder_at_context(F, lib, check, cfg, lay, small, head, ctx, room, stream, rng, kv_fmt=None):
    """A decoder over the stack with `ctx` earlier tokens' keys and values (synthetic) in every layer's cache and an input set.
    kv_fmt: block-quantized caches of that format instead of f32 ones."""
    from ferric_amd import decode as X
    nkv, hd, d = cfg.n_head_kv, cfg.head_dim, cfg.d_model
    dec = X.Qwen3Decoder(cfg, lay, max_len=ctx + room + 2, stream=stream, output_norm=small, lm_head=head, kv_fmt=kv_fmt)
    kv_fill = (rng.standard_normal((ctx, nkv * hd)) * 0.5).astype(np.float32)
    if kv_fmt is not None:
        kq = dec.caches[0][0]                     # quantized once, the packed arrays copied on the device
        kq.append(F.Tensor.from_vec(kv_fill, kv_fill.shape))
        check(lib.fhip_stream_sync(None))
        from ferric_amd import kvquant
        cw, sw = kvquant.sizes(kv_fmt, ctx, nkv * hd)
        for pair in dec.caches:
            for c in pair:
                if c is not kq:
                    check(lib.fhip_memcpy_d2d(c.codes.ptr, kq.codes.ptr, cw * 4, None))
                    check(lib.fhip_memcpy_d2d(c.scales.ptr, kq.scales.ptr, sw * 4, None))
        check(lib.fhip_stream_sync(None))
        dec.set_pos(ctx)
        dec.set_input((rng.standard_normal(d) * 0.5).astype(np.float32))
        return dec
    first = dec.caches[0]                         # uploaded once, copied on the device
    check(lib.fhip_memcpy_h2d(first.k.buf.ptr, kv_fill.ctypes.data_as(C.c_void_p), kv_fill.nbytes, None))
    check(lib.fhip_stream_sync(None))
    for c in dec.caches:
        if c is not first:
            check(lib.fhip_memcpy_d2d(c.k.buf.ptr, first.k.buf.ptr, kv_fill.nbytes, None))
        check(lib.fhip_memcpy_d2d(c.v.buf.ptr, first.k.buf.ptr, kv_fill.nbytes, None))
    check(lib.fhip_stream_sync(None))
    dec.set_pos(ctx)
    dec.set_input((rng.standard_normal(d) * 0.5).astype(np.float32))
    return dec


def bench_decode(F, lib, check, stream, timer, contexts=(128, 4096, 32768), layers=64, steps=6):
    """The decode weight sweep as a real decode step: the 64-layer stack of decode_stack(), with every op fed by the one before
    it: RMSNorm, q/k norm + rope + KV append, attention over `context` cached tokens (f32 cache), residual adds. One graph per
    step, replayed `steps` times at consecutive positions."""
    cfg, lay, small, head, weight_bytes_total, stacks = decode_stack(F, lib, check, layers)
    nkv, hd = cfg.n_head_kv, cfg.head_dim
    rng = np.random.default_rng(9)
    out = {}
    for ctx in contexts:
        dec = decoder_at_context(F, lib, check, cfg, lay, small, head, ctx, steps, stream, rng)
        dec.capture()
        dec.step_graph()                          # warm-up step (also: instantiation costs)
        ms = timer.time_ms(lambda: [dec.step_graph() for _ in range(steps)]) / steps
        logits = dec.logits.to_vec(stream)
        kv_bytes = 2 * (ctx + steps // 2) * nkv * hd * 4 * layers
        out[str(ctx)] = {"ms_per_token": ms, "tokens_per_s": 1e3 / ms, "launches_per_token": layers * dec.launches_per_layer + dec.launches_per_token_extra,
                         "kv_bytes_read": kv_bytes, "GBps_weights_plus_kv": (weight_bytes_total + kv_bytes) / (ms * 1e-3) / 1e9,
                         "logits_finite": bool(np.isfinite(logits).all())}
        del dec
    # the figures above are on weight handles as the library makes them (24-bit activations in the mat-vecs); the same step
    # with the handles switched to 16-bit activations, the precision `value` is quoted on
    def set_bits(bits):
        for L in lay:
            for w in (L.wqkv, L.wo, L.ffn_gate_up, L.ffn_down):
                w.matvec_precision(bits)
        head.matvec_precision(bits)
    set_bits(16)
    for ctx in contexts[:2]:
        dec = decoder_at_context(F, lib, check, cfg, lay, small, head, ctx, steps, stream, rng)
        dec.capture()
        dec.step_graph()
        ms = timer.time_ms(lambda: [dec.step_graph() for _ in range(steps)]) / steps
        out[str(ctx)]["ms_per_token_x16"] = ms
        del dec
    set_bits(24)
    out["activation_bits"] = 24
    # the same step on a Q8_0 block-quantized cache, attention reading the blocks in place (8.5 bits per cached value)
    ctx = contexts[-1]
    dec = decoder_at_context(F, lib, check, cfg, lay, small, head, ctx, steps, stream, rng, kv_fmt=0)
    dec.capture()
    dec.step_graph()
    ms = timer.time_ms(lambda: [dec.step_graph() for _ in range(steps)]) / steps
    logits = dec.logits.to_vec(stream)
    kv_bytes = 2 * (ctx + steps // 2) * (nkv * hd // 32) * 34 * layers
    out[f"{ctx}_q8_0_cache"] = {"ms_per_token": ms, "tokens_per_s": 1e3 / ms, "launches_per_token": layers * dec.launches_per_layer + dec.launches_per_token_extra,
                                "kv_bytes_read": kv_bytes, "logits_finite": bool(np.isfinite(logits).all())}
    del dec
    # the same stack on a block of prompt rows: projections on the bf16 matrix cores, causal attention on the f32 ones
    from ferric_amd import decode as X
    import time
    pre = {}
    for t in (512, 2048):
        dec = X.Qwen3Decoder(cfg, lay, max_len=t + 1, stream=stream)
        xs = (rng.standard_normal((t, cfg.d_model)) * 0.5).astype(np.float32)
        dec.prefill(xs[:64])                      # warm-up (first-use costs), then from an empty cache again
        dec.set_pos(0)
        check(lib.fhip_stream_sync(stream.handle))
        t0 = time.perf_counter()
        hid = dec.prefill(xs)                     # returns after the device has finished (it downloads the hidden rows)
        ms = (time.perf_counter() - t0) * 1e3
        pre[str(t)] = {"ms": ms, "tokens_per_s": t / (ms * 1e-3), "hidden_finite": bool(np.isfinite(hid).all())}
        del dec
    out["prefill_block"] = pre
    out["weight_bytes"] = weight_bytes_total
    out["model"] = "64 layers, d 5120, 40 query / 8 KV heads x 128, n_ff 17408, vocab 151936; Q4_K projections, Q6_K down and lm_head; f32 KV cache (the _q8_0_cache entry: Q8_0 blocks)"
    return out


def probe_step(F, lib, check):
    """Work for a kernel trace of the chained decode step without graph replay: the 64-layer decoder of bench_decode, three
    steps enqueued eagerly at context 128 and three at context 4096 (every launch of a step on the decoder's stream, in the
    order the captured graph holds them)."""
    stream = F.Stream()
    cfg, lay, small, head, _, stacks = decode_stack(F, lib, check, 64)
    rng = np.random.default_rng(9)
    for ctx in (128, 4096):
        dec = decoder_at_context(F, lib, check, cfg, lay, small, head, ctx, 4, stream, rng)
        for _ in range(3):
            dec.step()
        check(lib.fhip_stream_sync(stream.handle))
        assert np.isfinite(dec.logits.to_vec(stream)).all()
        del dec


def bench_prefill(F, lib, check, stream, timer, ts=(128, 512, 2048), reps=10):
    """Prefill: W 5120x5120 Q4_K, X [T, 5120] bf16 -> f32 [T, 5120] on the matrix cores; and the same on the
    layer's largest projection (fused gate|up, 34816x5120), where the launch has enough tiles to fill the chip."""
    from ferric_amd.synth import synth_weights
    res = {}
    for name, n, k in (("5120x5120", 5120, 5120), ("34816x5120", 34816, 5120)):
        qm = F.QMatrix.from_bytes(synth_weights(Q4_K, n, k, 1), Q4_K, n, k)
        out = {}
        for t in ts:
            xf = np.random.default_rng(7).standard_normal((t, k)).astype(np.float32)
            u = xf.view(np.uint32).astype(np.uint64)
            xb = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
            x = F.Tensor.from_bf16_bits(xb, (t, k))
            y = F.Tensor.empty((t, n))
            check(lib.fhip_workspace_reserve(stream.handle, lib.fhip_workspace_bytes_coop(qm.handle, None, t)))
            g = F.Graph.begin(stream)
            for _ in range(reps):
                check(lib.fhip_gemm_q_bf16(qm.handle, x.buf.ptr, t, y.buf.ptr, stream.handle))
            g.end()
            g.launch()
            ms = timer.steady_ms(g.launch) / reps
            tf = 2.0 * t * n * k / (ms * 1e-3) / 1e12
            out[str(t)] = {"ms": ms, "TFLOPs": tf, "frac_of_bf16_mfma_peak": tf / 2500.0}
            if t == max(ts):
                # The same launches (same graph, same instruction stream) on activations that are all zero: the difference is
                # what the switching activity of the operands costs in clock, i.e. how far the kernel is power-bound.
                check(lib.fhip_memset(x.buf.ptr, 0, 2 * t * k, stream.handle))
                g.launch()
                ms0 = timer.steady_ms(g.launch) / reps
                out[str(t)]["ms_on_zero_activations"] = ms0
        res[name] = out
    # What the matrix pipe gives with nothing else to do (register-resident operands, random mantissas), in graphs of ten
    # launches like the GEMMs above, at two launch lengths: about the 5120 x 5120 T = 2048 launch and about the large one.
    # The clock under sustained matrix work is set by the power limit, so this, not the 2.5 PFLOP/s at 2.4 GHz, is what
    # 100 % reads in wall-clock terms on this box.
    sink = F.DeviceBuffer(256)
    ceil = {}
    for label, iters in (("launch_of_130us", 900), ("launch_of_700us", 5000)):
        fl = C.c_double()
        g = F.Graph.begin(stream)
        for _ in range(reps):
            check(lib.fhip_debug_mfma_probe(iters, sink.ptr, C.byref(fl), stream.handle))
        g.end()
        g.launch()
        ms = timer.steady_ms(g.launch) / reps
        ceil[label] = {"ms": ms, "TFLOPs": fl.value / (ms * 1e-3) / 1e12}
    res["timing"] = "median of 5 replays of a graph of 10 launches, after >= 20 ms of the same replays"
    res["mfma_only_ceiling_TFLOPs"] = ceil["launch_of_700us"]["TFLOPs"]
    res["mfma_only_ceiling"] = ceil
    big = res["34816x5120"][str(max(ts))]
    big["frac_of_mfma_only_ceiling"] = big["TFLOPs"] / ceil["launch_of_700us"]["TFLOPs"]
    small = res["5120x5120"][str(max(ts))]
    small["frac_of_mfma_only_ceiling"] = small["TFLOPs"] / ceil["launch_of_130us"]["TFLOPs"]
    return res


def bench_prefill_attention(F, lib, check, stream, timer, reps=5):
    """Causal attention of a prompt block (fhip_causal_attention, f32 matrix instructions): 40 query / 8 KV heads x 128, T rows
    against a cache of S rows. FLOPs = 4 * head_dim * n_head * (query, key) pairs inside the causal mask."""
    nh, nkv, hd = 40, 8, 128
    rng = np.random.default_rng(1)
    out = {}
    for t, s in ((512, 512), (2048, 2048), (4096, 4096), (512, 8192)):
        q = F.Tensor.from_vec(rng.standard_normal((t, nh * hd)).astype(np.float32), (t, nh * hd))
        k = F.Tensor.from_vec(rng.standard_normal((s, nkv * hd)).astype(np.float32), (s, nkv * hd))
        v = F.Tensor.from_vec(rng.standard_normal((s, nkv * hd)).astype(np.float32), (s, nkv * hd))
        o = F.Tensor.empty((t, nh * hd))
        g = F.Graph.begin(stream)
        for _ in range(reps):
            check(lib.fhip_causal_attention(q.buf.ptr, k.buf.ptr, v.buf.ptr, t, s, nh, nkv, hd, 0, 0.0, o.buf.ptr, stream.handle))
        g.end()
        g.launch()
        ms = timer.steady_ms(g.launch) / reps
        pairs = t * (s - t) + t * (t + 1) / 2
        tf = 4.0 * pairs * nh * hd / (ms * 1e-3) / 1e12
        out[f"{t}x{s}"] = {"ms": ms, "TFLOPs": tf, "frac_of_f32_mfma_peak": tf / 157.3}
    return out


def probe(F, lib, check):
    """Work for a profiler run (kernel trace or hardware counters) of the mat-vec kernels, launched eagerly on the null stream:
    a copy of known size first (it calibrates FETCH_SIZE / WRITE_SIZE), then every weight shape of the decode sweep and the
    Q8_0 4096 x 4096 weight, each on rotating copies that add up to more than the 256 MB Infinity Cache so that every launch
    reads HBM: 512 launches of the headline Q4_K 5120 x 5120 (the O projection's shape too) over 64 copies, 256 of the fused
    QKV 7168 x 5120 over 40, 64 of gate|up 34816 x 5120 with SwiGLU over 8, 64 of down 5120 x 17408 Q6_K over 10, 512 of Q8_0
    4096 x 4096 over 56 and 8 of the vocabulary head 151936 x 5120 Q6_K over 2. The launches of a shape are enqueued back to
    back from native code (fhip_debug_matmul_q_loop), so the device sees the steady stream a captured graph would give it.
    Every shape runs twice: with 16-bit activations (what `value` is quoted on), then with 24-bit ones (what a new handle has)."""
    from ferric_amd.synth import synth_weights
    n = 256 << 20
    src, dst = F.DeviceBuffer(n), F.DeviceBuffer(n)
    check(lib.fhip_memset(src.ptr, 1, n, None))
    check(lib.fhip_stream_sync(None))
    check(lib.fhip_memcpy_d2d(dst.ptr, src.ptr, n, None))          # calibration dispatch: reads n, writes n
    check(lib.fhip_stream_sync(None))
    x = F.Tensor.from_vec(np.random.default_rng(2).standard_normal(5120).astype(np.float32), (1, 5120))
    x4 = F.Tensor.from_vec(np.random.default_rng(2).standard_normal(4096).astype(np.float32), (1, 4096))
    h = F.Tensor.from_vec(np.random.default_rng(3).standard_normal(17408).astype(np.float32), (1, 17408))
    y = F.Tensor.empty((1, 151936))
    plan = [(Q4_K, 5120, 5120, 64, 512, x, False), (Q4_K, 7168, 5120, 40, 256, x, False), (Q4_K, 34816, 5120, 8, 64, x, True),
            (Q6_K, 5120, 17408, 10, 64, h, False), (Q8_0, 4096, 4096, 56, 512, x4, False), (Q6_K, 151936, 5120, 2, 8, x, False)]
    for ty, rows, cols, ncopy, launches, xin, swiglu in plan:
        host = synth_weights(ty, rows, cols, 1)
        buf = replicate(F, lib, check, host, ncopy)
        ws = [F.QMatrix.wrap_device(buf, host.size, ty, rows, cols, offset=i * host.size) for i in range(ncopy)]
        handles = (C.c_void_p * ncopy)(*[w.handle for w in ws])
        for bits in (16, 24):       # the kernels carry the precision in their names: ..._p2 (16-bit activations), ..._p3 (24)
            for w in ws:
                w.matvec_precision(bits)
            check(lib.fhip_debug_matmul_q_loop(handles, ncopy, launches, xin.buf.ptr, 1 if swiglu else 0, y.buf.ptr, None))
            check(lib.fhip_stream_sync(None))
        del ws, buf


def probe_prefill(F, lib, check):
    """Work for a profiler run of the matrix-core kernels: Q4_K 5120x5120 and 34816x5120 at T = 2048 (tiled kernel),
    T = 128 (tiled, K split) and T = 8 (the T <= 32 kernel), 5 launches each; last, 5 more launches of 34816x5120 at
    T = 2048 on activations that are all zero (the same instruction stream with idle multipliers: what the clock does)."""
    from ferric_amd.synth import synth_weights
    for n, k in ((5120, 5120), (34816, 5120)):
        qm = F.QMatrix.from_bytes(synth_weights(Q4_K, n, k, 1), Q4_K, n, k)
        for t in (2048, 128, 8):
            xb = (np.random.default_rng(7).standard_normal((t, k)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
            x = F.Tensor.from_bf16_bits(xb, (t, k))
            y = F.Tensor.empty((t, n))
            for _ in range(5):
                check(lib.fhip_gemm_q_bf16(qm.handle, x.buf.ptr, t, y.buf.ptr, None))
            check(lib.fhip_stream_sync(None))
    t = 2048
    x = F.Tensor.from_bf16_bits(np.zeros((t, k), np.uint16), (t, k))
    y = F.Tensor.empty((t, n))
    for _ in range(5):
        check(lib.fhip_gemm_q_bf16(qm.handle, x.buf.ptr, t, y.buf.ptr, None))
    check(lib.fhip_stream_sync(None))


def probe_f16x2(F, lib, check, ncopy=4):
    """Work for a profiler run of the small-batch f16 matrix-core path at 8 activation rows: fhip_matmul_q_f16x2 on the
    gate|up (34816 x 5120 Q4_K) and down (5120 x 17408 Q6_K) weights, then the whole block through fhip_ffn_f16x2 and through
    fhip_ffn (ordered sums), 12 launches each, eagerly on the null stream, rotating over 4 copies of each weight (694 MB in all, more than the
    Infinity Cache holds) so that every launch reads HBM. Last, 32 launches of fhip_matmul_q_f16x2 over 32 copies of a
    4096 x 4096 Q8_0 weight (571 MB) and 16 over 16 copies of a 12288 x 4096 one (857 MB), 8 rows each. Between the two: 12
    launches of fhip_ffn at 4 rows (gate|up + SwiGLU on the four-row mat-vec, down on the f16 kernels) and 12 with the weights
    set to FHIP_BATCH_F32_MATVEC (both on the four-row mat-vec)."""
    from ferric_amd.synth import synth_weights
    n_embd, n_ff, t = 5120, 17408, 8
    gbuf = replicate(F, lib, check, synth_weights(Q4_K, 2 * n_ff, n_embd, 3), ncopy)
    dbuf = replicate(F, lib, check, synth_weights(Q6_K, n_embd, n_ff, 4), ncopy)
    gb, db = weight_bytes(Q4_K, 2 * n_ff, n_embd), weight_bytes(Q6_K, n_embd, n_ff)
    gus = [F.QMatrix.wrap_device(gbuf, gb, Q4_K, 2 * n_ff, n_embd, offset=i * gb) for i in range(ncopy)]
    dns = [F.QMatrix.wrap_device(dbuf, db, Q6_K, n_embd, n_ff, offset=i * db) for i in range(ncopy)]
    rng = np.random.default_rng(5)
    x = F.Tensor.from_vec(rng.standard_normal((t, n_embd)).astype(np.float32), (t, n_embd))
    h = F.Tensor.from_vec(rng.standard_normal((t, n_ff)).astype(np.float32), (t, n_ff))
    for ws_, xin in ((gus, x), (dns, h)):
        y = F.Tensor.empty((t, ws_[0].rows()))
        ws = F.DeviceBuffer(lib.fhip_matmul_q_f16x2_ws_bytes(ws_[0].handle, t))
        for i in range(12):
            check(lib.fhip_matmul_q_f16x2(ws_[i % ncopy].handle, xin.buf.ptr, t, y.buf.ptr, ws.ptr, None))
        check(lib.fhip_stream_sync(None))
    y = F.Tensor.empty((t, n_embd))
    ws = F.DeviceBuffer(lib.fhip_ffn_f16x2_ws_bytes(gus[0].handle, dns[0].handle, t))
    for i in range(12):
        check(lib.fhip_ffn_f16x2(gus[i % ncopy].handle, dns[i % ncopy].handle, x.buf.ptr, t, y.buf.ptr, ws.ptr, None))
    check(lib.fhip_stream_sync(None))
    # the drop-in call on the same weights: handles as the library makes them add the partial sums of cut rows in a fixed
    # order (FHIP_BATCH_ORDERED) instead of atomically, gate|up's inside the split for the down projection
    hws = F.Tensor.empty((t, n_ff))
    for i in range(12):
        check(lib.fhip_ffn(gus[i % ncopy].handle, dns[i % ncopy].handle, x.buf.ptr, t, y.buf.ptr, hws.buf.ptr, None))
    check(lib.fhip_stream_sync(None))
    # four rows: fhip_ffn runs gate|up + SwiGLU on the four-row mat-vec (the int8 4 x 4 x 4 matrix instruction) and the down
    # projection on the f16 kernels; then the same call with every row on the mat-vec's arithmetic (FHIP_BATCH_F32_MATVEC)
    x4 = F.Tensor.from_vec(np.random.default_rng(5).standard_normal((4, n_embd)).astype(np.float32), (4, n_embd))   # (bench_ffn's rows)
    y4 = F.Tensor.empty((4, n_embd))
    for policy in (2, 1):
        for w in gus + dns:
            w.batch_policy(policy)
        for i in range(12):
            check(lib.fhip_ffn(gus[i % ncopy].handle, dns[i % ncopy].handle, x4.buf.ptr, 4, y4.buf.ptr, hws.buf.ptr, None))
        check(lib.fhip_stream_sync(None))
    del gus, dns, gbuf, dbuf
    for rows, nc in ((4096, 32), (12288, 16)):
        nb = weight_bytes(Q8_0, rows, 4096)
        qbuf = replicate(F, lib, check, synth_weights(Q8_0, rows, 4096, 0), nc)
        x8 = F.Tensor.from_vec(rng.standard_normal((t, 4096)).astype(np.float32), (t, 4096))
        y8 = F.Tensor.empty((t, rows))
        ws8 = None
        for i in range(nc):
            w = F.QMatrix.wrap_device(qbuf, nb, Q8_0, rows, 4096, offset=i * nb)
            ws8 = ws8 or F.DeviceBuffer(lib.fhip_matmul_q_f16x2_ws_bytes(w.handle, t))
            check(lib.fhip_matmul_q_f16x2(w.handle, x8.buf.ptr, t, y8.buf.ptr, ws8.ptr, None))
        check(lib.fhip_stream_sync(None))


def probe_decode(F, lib, check):
    """Work for a hardware-counter run on the decode attention kernel: a copy of known size (calibrates FETCH_SIZE /
    WRITE_SIZE), then 8 launches of fhip_decode_attention on 8 different caches of 4096 rows (40 query / 8 KV heads x 128:
    33.6 MB of K and V rows each, none touched before), then 8 at 128 rows."""
    from ferric_amd import decode as X
    n = 256 << 20
    src, dst = F.DeviceBuffer(n), F.DeviceBuffer(n)
    check(lib.fhip_memset(src.ptr, 1, n, None))
    check(lib.fhip_stream_sync(None))
    check(lib.fhip_memcpy_d2d(dst.ptr, src.ptr, n, None))
    check(lib.fhip_stream_sync(None))
    nh, nkv, hd = 40, 8, 128
    rng = np.random.default_rng(3)
    fill = (rng.standard_normal((4096, nkv * hd)) * 0.5).astype(np.float32)
    caches = []
    for _ in range(8):
        c = X.KvCache(4096, nkv * hd)
        check(lib.fhip_memcpy_h2d(c.k.buf.ptr, fill.ctypes.data_as(C.c_void_p), fill.nbytes, None))
        check(lib.fhip_memcpy_h2d(c.v.buf.ptr, fill.ctypes.data_as(C.c_void_p), fill.nbytes, None))
        c.len = 4096
        caches.append(c)
    check(lib.fhip_stream_sync(None))
    check(lib.fhip_memcpy_d2d(dst.ptr, src.ptr, n, None))          # pushes the freshly written caches out of the cache levels
    check(lib.fhip_stream_sync(None))
    q = F.Tensor.from_vec(rng.standard_normal(nh * hd).astype(np.float32), (1, nh * hd))
    for length in (4096, 128):
        for c in caches:
            X.decode_attention(q, c, nh, nkv, length=length)
    check(lib.fhip_stream_sync(None))


def probe_prefill_attn(F, lib, check):
    """Work for a profiler run on the causal attention kernel: 40 query / 8 KV heads x 128, five launches each at 2048 rows
    against 2048 (a stateless prefill), at 512 against 512 and at 512 against a cache of 8192 (a chunk of a long prompt)."""
    from ferric_amd import decode as X
    nh, nkv, hd = 40, 8, 128
    rng = np.random.default_rng(1)
    for t, s in ((2048, 2048), (512, 512), (512, 8192)):
        q = F.Tensor.from_vec(rng.standard_normal((t, nh * hd)).astype(np.float32), (t, nh * hd))
        k = F.Tensor.from_vec(rng.standard_normal((s, nkv * hd)).astype(np.float32), (s, nkv * hd))
        v = F.Tensor.from_vec(rng.standard_normal((s, nkv * hd)).astype(np.float32), (s, nkv * hd))
        for _ in range(5):
            X.causal_attention(q, k, v, nh, nkv)
    check(lib.fhip_stream_sync(None))


def probe_kvq(F, lib, check):
    """Work for a kernel trace of attention over a long cache: 40 query / 8 KV heads x 128 at 32768 cached rows, four launches
    each on four f32 caches (268 MB of rows per launch) and on four caches of every block format (71 / 38 / 42 MB), every
    cache read for the first time by its launch; then one token's K and V rows appended to a quantized cache four times."""
    from ferric_amd import decode as X
    from ferric_amd import kvquant as Q
    nh, nkv, hd, rows = 40, 8, 128, 32768
    rng = np.random.default_rng(3)
    fill = (rng.standard_normal((rows, nkv * hd)) * 0.5).astype(np.float32)
    ft = F.Tensor.from_vec(fill, fill.shape)
    q = F.Tensor.from_vec(rng.standard_normal(nh * hd).astype(np.float32), (1, nh * hd))
    plain = []
    for _ in range(4):
        c = X.KvCache(rows, nkv * hd)
        check(lib.fhip_memcpy_d2d(c.k.buf.ptr, ft.buf.ptr, fill.nbytes, None))
        check(lib.fhip_memcpy_d2d(c.v.buf.ptr, ft.buf.ptr, fill.nbytes, None))
        c.len = rows
        plain.append(c)
    packed = {fmt: [(Q.QKvCache.from_tensor(ft, fmt), Q.QKvCache.from_tensor(ft, fmt)) for _ in range(4)] for fmt in Q.ALL}
    check(lib.fhip_stream_sync(None))
    scrub_src, scrub_dst = F.DeviceBuffer(512 << 20), F.DeviceBuffer(512 << 20)
    check(lib.fhip_memcpy_d2d(scrub_dst.ptr, scrub_src.ptr, 512 << 20, None))      # pushes what was just written out of the cache levels
    check(lib.fhip_stream_sync(None))
    for c in plain:
        X.decode_attention(q, c, nh, nkv)
    for fmt in Q.ALL:
        for kq, vq in packed[fmt]:
            X.decode_attention_kvq(q, kq, vq, nh, nkv)
    row = F.Tensor.from_vec(fill[:1], (1, nkv * hd))
    kq, vq = Q.QKvCache(Q.Q8_0, 64, nkv * hd), Q.QKvCache(Q.Q8_0, 64, nkv * hd)
    for i in range(4):
        check(lib.fhip_kvq_append2(Q.Q8_0, row.buf.ptr, row.buf.ptr, 0, 1, nkv * hd, None, i, 64, kq.codes.ptr, kq.scales.ptr, vq.codes.ptr,
                                   vq.scales.ptr, None))
    check(lib.fhip_stream_sync(None))


def cpu_baseline(rows, cols, x_seed, budget_s=12.0):
    """The reference's CPU route for Q4_K (deq_raw then a sequential f32 dot per row, rows split in
    contiguous spans over threads), timed through the C oracle on this host's cores."""
    from ferric_amd.synth import synth_weights
    from oracle import oracle as O
    O.build()
    try:
        avail = len(os.sched_getaffinity(0))
    except AttributeError:
        avail = os.cpu_count() or 1
    threads = max(1, min(16, avail))          # the GPU box's CPU share is 16 threads, whatever the host shows
    w = synth_weights(Q4_K, rows, cols, 1)
    x = np.random.default_rng(x_seed).standard_normal(cols).astype(np.float32)
    O.matmul_cpu(x, w, Q4_K, rows, cols, threads=threads)  # warm-up, excluded
    times, t_end = [], time.perf_counter() + budget_s
    while len(times) < 9 or (time.perf_counter() < t_end and len(times) < 1000):
        t0 = time.perf_counter()
        O.matmul_cpu(x, w, Q4_K, rows, cols, threads=threads)
        times.append(time.perf_counter() - t0)
        if time.perf_counter() > t_end and len(times) >= 9:
            break
    med = float(np.median(times))
    alg = w.size + 4 * cols + 4 * rows
    return {"value": alg / med / 1e9, "unit": "GB/s", "cores": threads, "host_logical_cpus": os.cpu_count(), "kind": "port",
            "sample": f"{len(times)} full Q4_K 5120x5120 batch-1 mat-vecs (dequantize row, then sequential f32 dot; "
                      f"contiguous row spans over {threads} threads), median {med * 1e3:.2f} ms each"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=64)
    ap.add_argument("--no-sweep", action="store_true")
    ap.add_argument("--no-ffn", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-q8", action="store_true")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-moe", action="store_true")
    ap.add_argument("--no-decode", action="store_true")
    ap.add_argument("--headline-only", action="store_true",
                    help="only the cold-rotation Q4_K 5120x5120 GEMV loop (what `value` is computed from); for profiling")
    ap.add_argument("--probe", action="store_true",
                    help="counter probe for rocprofv3 --pmc: one 256 MiB device copy (calibration), then 16 cold Q4_K 5120x5120 "
                         "GEMVs, one fused gate|up 34816x5120 and one Q6_K 5120x17408 GEMV; prints nothing else")
    ap.add_argument("--probe-step", action="store_true", help="three eager decode steps at context 128 and 4096 (for a kernel trace)")
    ap.add_argument("--probe-prefill-attn", action="store_true", help="causal attention at 2048 / 512 rows (for a profiler run)")
    ap.add_argument("--probe-kvq", action="store_true", help="attention at 32768 rows on f32 and block-quantized caches (for a kernel trace)")
    ap.add_argument("--probe-decode", action="store_true",
                    help="profiler probe for the decode attention kernel: 8 launches each at 4096 and 128 cached rows; prints nothing else")
    ap.add_argument("--probe-prefill", action="store_true",
                    help="profiler probe for the matrix-core GEMM: Q4_K 5120x5120 and 34816x5120 at T = 2048, 128 and 8, "
                         "5 launches each; prints nothing else")
    ap.add_argument("--probe-f16x2", action="store_true",
                    help="profiler probe for the small-batch f16 matrix-core path: gate|up, down and the whole FFN block at 8 "
                         "rows, 5 launches each; prints nothing else")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (--gpus 1); multi-GPU sharding is a design note, not code")

    import ferric_amd as F
    from ferric_amd import _lib
    lib = _lib.init(0)
    check = _lib.check
    stream = F.Stream()
    timer = Timer(lib, check, stream)

    rows = cols = 5120
    if args.probe:
        probe(F, lib, check)
        return
    if args.probe_f16x2:
        probe_f16x2(F, lib, check)
        return
    if args.probe_prefill:
        probe_prefill(F, lib, check)
        return
    if args.probe_kvq:
        probe_kvq(F, lib, check)
        return
    if args.probe_prefill_attn:
        probe_prefill_attn(F, lib, check)
        return
    if args.probe_decode:
        probe_decode(F, lib, check)
        return
    if args.probe_step:
        probe_step(F, lib, check)
        return
    log("[bench] Q4_K GEMV 5120x5120 ...")
    # `value`: handles switched to 16-bit activations (QMatrix.matvec_precision(16)): inside the benchmark's tolerance
    # 1e-3 * ||w_row|| * ||x|| by three orders of magnitude, but not inside the 1e-5 of the reference's own examples. A handle as
    # the library makes it computes at 24 bits (the f32 significand, which those examples pass): `value_x24` beside it.
    c2, alg, nbytes = bench_gemv(F, lib, check, stream, timer, Q4_K, rows, cols, args.steps, args.warmup, seed=1, x_seed=2, ncopy=64,
                                 cold_only=args.headline_only, with_reader=True, bits=16)
    x24 = None
    if args.headline_only:
        args.no_q8 = args.no_ffn = args.no_prefill = args.no_moe = args.no_sweep = args.no_cpu = args.no_decode = True
        c2["warm"] = None
    else:
        x24, _, _ = bench_gemv(F, lib, check, stream, timer, Q4_K, rows, cols, args.steps, args.warmup, seed=1, x_seed=2, ncopy=64, bits=24)
    ms_step = c2["cold"]["ms_per_step"]
    value = c2["cold"]["GBps"]
    traffic = headline_traffic()
    line = {
        "metric": "Q4_K GEMV HBM GB/s (% of 8 TB/s) at batch 1; decode-step weight-sweep ms",
        "value": value, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32 in / f32 out; weights Q4_K exact; activations inside the kernel: 16-bit block fixed point per 32 columns (opt-in; "
                 "a new handle has 24-bit: value_x24), integer dot products per sub-block, f32 accumulation above it",
        "data": "synthetic",
        "config": {"workload": "Q4_K GEMV batch 1, W 5120x5120 (14745600 B raw GGUF blocks), x f32[5120]; "
                               "64 distinct weight copies rotated (944 MB > 256 MB Infinity Cache) so each step reads HBM",
                   "rows": rows, "cols": cols, "batch": 1, "weight_copies": 64},
        "pct_of_peak": 100.0 * value / HBM_PEAK_GBPS,
        "value_x16": value, "us_x16": ms_step * 1e3,
        "value_x24": x24["cold"]["GBps"] if x24 else None, "us_x24": x24["cold"]["ms_per_step"] * 1e3 if x24 else None,
        "warm_single_copy": c2["warm"],
        "roofline": {"bound": "hbm", "achieved": alg / (ms_step * 1e-3) / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": alg / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                     "traffic": traffic.get("hbm_bytes_per_launch") if traffic else None, "traffic_source": traffic,
                     "kernel": "gemv_stream_kernel<Q4K, M=1, plain>, two activation planes (16-bit)", "algorithmic_bytes_per_launch": alg,
                     "launch_us": ms_step * 1e3,
                     # the same 14.7 MB through a kernel that only reads them (same rotation, same timing), and a launch
                     # that does nothing: what this box leaves a single cold launch of this size
                     "reader_floor_us": c2["reader_ms"] * 1e3, "frac_of_reader": c2["reader_ms"] / ms_step,
                     "empty_launch_us": launch_floor_us(F, lib, check, stream, timer)},
        "activation_bits": 16,
        "timing": "median of 9 batches; a batch = the K-step graph(s) replayed back to back until >= 1024 launches, one HIP event pair",
    }
    if not args.headline_only:
        log("[bench] time against bytes (fixed cost and marginal rate) ...")
        fit = bench_marginal(F, lib, check, stream, timer)
        line["roofline"]["marginal_GBps"] = fit["mat_vec"]["marginal_GBps"]
        line["roofline"]["marginal_frac"] = fit["mat_vec"]["marginal_frac_of_peak"]
        line["roofline"]["fixed_us"] = fit["mat_vec"]["fixed_us"]
        line["roofline"]["time_vs_bytes"] = fit
    if not args.no_q8:
        log("[bench] Q8_0 GEMV 4096x4096 ...")
        c1, alg1, _ = bench_gemv(F, lib, check, stream, timer, Q8_0, 4096, 4096, args.steps, args.warmup, seed=0, x_seed=0, ncopy=56)
        line["q8_0_gemv_4096"] = {"cold_GBps": c1["cold"]["GBps"], "cold_us": c1["cold"]["ms_per_step"] * 1e3,
                                  "warm_GBps": c1["warm"]["GBps"], "algorithmic_bytes": alg1,
                                  "batch8": bench_q80_batch(F, lib, check, stream, timer)}
    if not args.no_ffn:
        log("[bench] Q4_K_M FFN block, batch 1/4/8 ...")
        ffn, wb = bench_ffn(F, lib, check, stream, timer, (1, 4, 8))
        line["ffn_q4k_q6k"] = {"weight_bytes": wb, "batch": ffn}
    if not args.no_prefill:
        log("[bench] prefill dequant-GEMM, T = 128/512/2048 ...")
        line["prefill_q4k_bf16_mfma"] = bench_prefill(F, lib, check, stream, timer)
        line["prefill_causal_attention_f32_mfma"] = bench_prefill_attention(F, lib, check, stream, timer)
    if not args.no_moe:
        log("[bench] routed-expert block of an MoE decode layer ...")
        line["moe_routed_experts_q4k_q6k"] = bench_moe(F, lib, check, stream, timer)
    if not args.no_moe:
        log("[bench] Q5_K / Q4_0 / Q4_1 / Q5_0 / Q5_1 / IQ4_NL / IQ4_XS / MXFP4 GEMV 5120x5120 ...")
        other = {}
        for name, ty in (("q5_k", 13), ("q4_0", 2), ("q4_1", 3), ("q5_0", 6), ("q5_1", 7), ("iq4_nl", 20), ("iq4_xs", 23), ("mxfp4", 39)):
            r, a, nb = bench_gemv(F, lib, check, stream, timer, ty, rows, cols, 64, 64, seed=20 + ty, x_seed=2, ncopy=48)
            other[name] = {"cold_us": r["cold"]["ms_per_step"] * 1e3, "cold_GBps": r["cold"]["GBps"],
                           "warm_us": r["warm"]["ms_per_step"] * 1e3, "algorithmic_bytes": a}
        line["other_formats_gemv_5120"] = other
    if not args.no_moe:
        log("[bench] GGUF ingest ...")
        line["gguf_ingest"] = bench_gguf(F, lib, check)
        line["host_buffer_entry_points"] = bench_host_entry(F)
    if not args.no_sweep:
        log("[bench] 64-layer decode weight sweep (14.0 GB) ...")
        line["decode_sweep"] = bench_sweep(F, lib, check, stream, timer)
        log("[bench] weight shapes of other models ...")
        line["other_model_shapes"] = bench_other_shapes(F, lib, check, stream, timer)
    if not args.no_decode:
        log("[bench] 64-layer decode step with attention (context 128 / 4096 / 32768) ...")
        line["decode_step_chained"] = bench_decode(F, lib, check, stream, timer)
    if not args.no_cpu:
        log("[bench] CPU baseline (oracle port) ...")
        line["cpu_baseline"] = cpu_baseline(rows, cols, 2)
    else:
        line["cpu_baseline"] = None
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
