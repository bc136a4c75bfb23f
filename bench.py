#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

One "step" is one launch of `incin_rocm_sdpa_fwd` over one batch of synthetic
input already resident in HBM.  The headline workload is BASELINE config 3
(bf16 causal prefill, B=8 H=16 S=4096 D=128); BASELINE config 4 (bf16 decode,
B=32 H=32 KV=8192 D=128, split-KV + combine) is measured in the same run and
reported under "decode".  The last line of stdout is ONE compact JSON line (the headline, its roofline and CPU
baseline, and the decode and ragged-prefill figures); every other leg is written in full to `bench_detail.json`
beside this file and echoed to stderr.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline]

Timing: K steps between two device synchronisations (wall clock -> ms_per_step,
value) and, for the roofline figure, HIP events recorded around every launch on
the stream the kernels run on (the library's event entry points).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from incin_amd import capi, dtypes, host  # noqa: E402

SEED0 = 20261125
PEAK_BF16_TFLOPS = 2516.6   # 256 CUs x 2.4 GHz x 4096 dense bf16 FLOP/clk/CU (vendor: 2.5 PFLOP/s)
PEAK_F32_TFLOPS = 157.3      # dense fp32 matrix peak, vendor figure (256 CUs x 2.4 GHz x 256 FLOP/clk/CU)
PEAK_HBM_GBS = 8000.0       # HBM3E, vendor figure
# HBM bytes per launch, from rocprofv3 --pmc runs of this same script, one leg (and where a leg has several shapes on one
# kernel, one shape) at a time: `rocprofv3 --pmc FETCH_SIZE -- python3 bench.py --only LEG [--shape NAME] --steps 10
# --warmup 2 --no-cpu-baseline`, then the same with WRITE_SIZE; KiB per dispatch, mean of the leg's last 20 dispatches of each
# kernel, the kernels of one launch (main + combine, the backward's three) added up.  The counters are calibrated against
# the 1 GiB copy kernel (`--only copy`: FETCH_SIZE 524294, WRITE_SIZE 1048580 KiB), hence FETCH_SIZE x 2.0, WRITE_SIZE x 1.0.
# These are constants taken from counter runs, not measured by this script: each roofline object says so and names the
# summary under profiles/ that records the run.
TRAFFIC_KIB = {   # leg/shape/variant: (FETCH_SIZE, WRITE_SIZE)
    "prefill": (263343, 131074),                           # 5.39e8 + 1.34e8: |O| written once, |Q|+|K|+|V| read 1.34 times
    "decode": (2097380, 256.0),                            # 4.295e9: K and V read once
    "decode/vector_alu": (2097460 + 616.5, 1088.2 + 256),
    "prefill_long": (453220, 318928),                      # valid |O| written once, the inputs read 1.9 times
    "decode_gqa/gqa4_b32_kv8192/auto": (524504, 256), "decode_gqa/gqa4_b32_kv8192/vector_alu": (525386 + 2152.5, 4352 + 256),
    "decode_gqa/gqa4_b32_kv8192/bias": (524760, 256),
    "decode_gqa/gqa4_b1_kv131072/auto": (262264 + 2120.5, 544 + 8), "decode_gqa/gqa4_b1_kv131072/vector_alu": (262250 + 2120.5, 4352.2 + 8),
    "decode_gqa/gqa8_b32_kv8192/auto": (524632, 512), "decode_gqa/gqa8_b32_kv8192/vector_alu": (526452 + 4264.5, 8704 + 512),
    "decode_gqa/gqa4_sq4_b8_kv8192/auto": (132176 + 2152.5, 4352.1 + 256),
    "decode_gqa/f32_gqa4_b32_kv8192/auto": (1048910, 512), "decode_gqa/f32_gqa4_b32_kv8192/vector_alu": (1050700 + 2152, 4352 + 512),
    "decode_gqa/f32_gqa8_sq4_b8_kv8192/auto": (266342 + 4264, 8704.3 + 1024),
    "head_dims/prefill_d96": (109157, 62546.7), "head_dims/prefill_d256": (556912, 131083), "head_dims/chunk_d256": (68960.5 + 33320.5, 67438.4 + 4096),
    "head_dims/decode_d96": (393400, 192), "head_dims/decode_d256": (1048960, 512), "head_dims/prefill_d96_s4096": (206387, 123320),
    "prefill_chunk/bf16_sq128_kv32768/auto": (66326.4 + 16680.5, 33392.9 + 1024), "prefill_chunk/bf16_sq128_kv32768/unsplit": (66199.5, 1024),
    "prefill_chunk/bf16_sq512_kv32768/auto": (67708 + 17448.5, 33677.2 + 4096), "prefill_chunk/bf16_sq512_kv32768/unsplit": (67735.5, 4096),
    "prefill_chunk/f32_sq128_kv32768/auto": (132204 + 16680, 33316.9 + 2048), "prefill_chunk/f32_sq128_kv32768/unsplit": (132192, 2048),
    "f32/f32_c1": (187.2, 32), "f32/f32_c2": (12378.4, 8192), "f32/f32_large": (1523050, 262144),
    "backward/bf16_d128": (133150 + 367216 + 264788, 4096 + 131072 + 262324),          # (row dots + dQ + dK/dV kernels)
    "backward/bf16_d64": (135199 + 309173 + 266324, 8192 + 131072 + 262152),
    # (config 2's shape in f32: blocks dealt to two workgroups - the kernels write a plane each beside the gradients, and the two
    #  passes that add the planes follow)
    "backward/f32_d64": (8735 + 16613 + 16883 + 8219 + 16411, 512 + 16384 + 32778.2 + 8192 + 16384),
    "backward/f32_d128": (270367 + 875814 + 924203, 8192 + 262144 + 524288),
}
TRAFFIC_PROFILE = "profiles/fetch_write_size_bench_legs.txt"


def traffic_of(key):
    """(HBM bytes per launch, where the figure comes from) for one leg / shape / variant of the table above."""
    if TRAFFIC_KIB.get(key) is None:
        return None, None
    fetch, write = TRAFFIC_KIB[key]
    return (fetch * 2.0 + write) * 1024.0, "constant from %s (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE of `bench.py --only %s`)" % (TRAFFIC_PROFILE, key.split("/")[0])


METRIC = "attn fwd TFLOP/s + % bf16 MFMA peak; decode KV GB/s + % HBM peak (1 GPU)"


def rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def make_inputs(seed, B, Hq, Hkv, Sq, Skv, D, dtype):
    r = rng(seed)
    q = r.standard_normal((B, Hq, Sq, D), dtype=np.float32)
    k = r.standard_normal((B, Hkv, Skv, D), dtype=np.float32)
    v = r.standard_normal((B, Hkv, Skv, D), dtype=np.float32)
    return q, k, v


def causal_flops(B, Hq, Sq, Skv, D):
    pairs = sum(min(max(i + 1 + Skv - Sq, 0), Skv) for i in range(Sq)) if Sq != Skv else Sq * (Sq + 1) // 2
    return 4.0 * D * B * Hq * pairs


class Workload:
    """Device-resident operands + descriptor for one configuration."""

    def __init__(self, name, seed, B, Hq, Hkv, Sq, Skv, D, dtype, causal, kv_lens=None, pad_queries=False, impl=capi.IMPL_AUTO, num_splits=0):
        self.name, self.shape = name, (B, Hq, Hkv, Sq, Skv, D)
        self.dtype, self.causal, self.kv_lens = dtype, causal, kv_lens
        q, k, v = make_inputs(seed, B, Hq, Hkv, Sq, Skv, D, dtype)
        self.host = (q, k, v)
        self.tq, self.tk, self.tv = (host.DeviceTensor.from_f32(x, dtype) for x in (q, k, v))
        self.to = host.DeviceTensor((B, Hq, Sq, D), dtype)
        self.tl = capi.DeviceBuffer.from_numpy(np.asarray(kv_lens, dtype=np.int32)) if kv_lens is not None else None
        # a padded self-attention batch: the same lengths say which keys and which query rows are padding
        self.desc = host.make_desc(self.tq, self.tk, self.tv, self.to, causal=causal, kv_lens=self.tl,
                                   q_lens=self.tl if pad_queries else None, impl=impl, num_splits=num_splits)
        self.descs, self.more_kv, self.turn = [self.desc], [], 0
        self._make_kw = dict(causal=causal, kv_lens=self.tl, q_lens=self.tl if pad_queries else None)
        self.ws = None
        self.replan(impl, num_splits)

    def rotate_kv(self, min_bytes=512 << 20):
        """Launches that read less than `min_bytes` of K and V take turns over as many copies of the cache as add up to
        that much: back-to-back launches over one small cache would be served by the 256 MB last-level cache, not by
        HBM, and a fraction of the HBM peak taken from them would mean nothing.  Returns the number of copies."""
        B, Hq, Hkv, Sq, Skv, D = self.shape
        kv_bytes = 2 * B * Hkv * Skv * D * (4 if self.dtype == capi.F32 else 2)
        n = min(8, -(-min_bytes // kv_bytes))
        for _ in range(n - len(self.descs)):
            tk, tv = (host.DeviceTensor.from_f32(x, self.dtype) for x in self.host[1:])
            self.more_kv += [tk, tv]
            self.descs.append(host.make_desc(self.tq, tk, tv, self.to, impl=self.desc.impl, num_splits=self.desc.num_splits, **self._make_kw))
        self.replan(self.desc.impl, self.desc.num_splits)
        return len(self.descs)

    def replan(self, impl=capi.IMPL_AUTO, num_splits=0):
        """The same operands through another kernel or split count (generating and uploading gigabytes of cache again
        would cost more than the measurement)."""
        if self.ws is not None:
            self.ws.free()
        for d in self.descs:
            d.impl, d.num_splits = impl, num_splits
            d.workspace, d.workspace_bytes = None, 0
        nbytes, self.splits, self.impl = capi.sdpa_workspace(self.desc)
        self.ws = capi.DeviceBuffer(nbytes) if nbytes else None
        if self.ws is not None:
            for d in self.descs:                 # (launches follow each other on one stream: one workspace serves every copy)
                d.workspace, d.workspace_bytes = self.ws.ptr, self.ws.nbytes

    def launch(self):
        capi.sdpa_fwd(self.descs[self.turn])
        self.turn = self.turn + 1 if self.turn + 1 < len(self.descs) else 0

    def ramp(self, seconds=0.15):
        """Setup, not measurement: keep the GPU busy until its clocks have settled (the first ~30 launches
        after idle run up to 40% slower), so that the W warm-up steps and the K timed steps see steady state."""
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < seconds:
            for _ in range(10):
                self.launch()
            capi.sync()

    def time(self, steps, warmup):
        """(wall ms per step over `steps` back-to-back launches, mean / median / min event ms per launch)"""
        self.ramp()
        for _ in range(warmup):
            self.launch()
        capi.sync()
        r0, r1 = capi.Event(), capi.Event()
        t0 = time.perf_counter()
        r0.record()
        for _ in range(steps):
            self.launch()
        r1.record()
        capi.sync()
        wall_ms = (time.perf_counter() - t0) * 1e3 / steps
        # the same K launches by the device's clock: two events around the whole timed region (for launches of tens of
        # microseconds, where an event pair around every launch adds microseconds of its own to each)
        self.region_ms = r0.elapsed_ms(r1) / steps
        r0.destroy()
        r1.destroy()
        starts = [capi.Event() for _ in range(steps)]
        stops = [capi.Event() for _ in range(steps)]
        for i in range(steps):
            starts[i].record()
            self.launch()
            stops[i].record()
        capi.sync()
        ev = np.array([starts[i].elapsed_ms(stops[i]) for i in range(steps)])
        for e in starts + stops:
            e.destroy()
        return wall_ms, float(ev.mean()), float(np.median(ev)), float(ev.min())

    def parity(self, n_rows=48):
        """max-abs error of sampled output rows against the CPU oracle (checker only)."""
        from oracle import oracle as O
        B, Hq, Hkv, Sq, Skv, D = self.shape
        G = Hq // Hkv
        q, k, v = (dtypes.round_to(x, self.dtype) for x in self.host)
        out = self.to.to_f32()
        r = rng(99)
        rows = np.stack([r.integers(0, B * Hq, n_rows), r.integers(0, Sq, n_rows)], axis=1)
        rows[0] = (0, 0)
        rows[1] = (B * Hq - 1, Sq - 1)
        lens = None
        if self.kv_lens is not None:       # sample inside each sequence's valid length (rows past it are padding queries)
            lens = np.asarray(self.kv_lens, dtype=np.int32)
            rows[:, 1] %= lens[rows[:, 0] // Hq]
            lens = lens.reshape(B, 1, 1)
        ref = O.sdpa_rows(q.reshape(B, Hkv, G, Sq, D), k[:, :, None], v[:, :, None], rows, causal=self.causal, kv_lens=lens)
        got = out.reshape(B * Hq, Sq, D)[rows[:, 0], rows[:, 1]]
        return float(np.abs(got - ref).max())

    def free(self):
        for t in [self.tq.buf, self.tk.buf, self.tv.buf, self.to.buf, self.ws, self.tl] + [x.buf for x in self.more_kv]:
            if t is not None:
                t.free()


def launch_duration(w, ev_mean):
    """(ms per launch, how it was taken): launches under 0.2 ms by two HIP events around the timed region of K launches
    (an event pair around every launch adds microseconds of its own to each), longer ones by the mean of the pairs."""
    if ev_mean < 0.2:
        return w.region_ms, "two HIP events around the timed launches"
    return ev_mean, "an event pair around each launch"


def cpu_baseline_prefill(D, S, slices, dtype):
    """The oracle's materialising form (the reference's execution shape: serial matmuls and
    reductions, threaded elementwise maps) on `slices` (b,h) slices of the causal-prefill workload."""
    from oracle import oracle as O
    q, k, v = make_inputs(SEED0 + 2, 1, slices, slices, S, S, D, dtype)
    q, k, v = (dtypes.round_to(x, dtype) for x in (q, k, v))
    mask = O.causal_additive_mask(S, S)
    t0 = time.perf_counter()
    O.sdpa_materialised(q, k, v, mask=mask)
    dt = time.perf_counter() - t0
    return causal_flops(1, slices, S, S, D) / dt / 1e12, dt


def host_cpu():
    """CPU model name and logical CPU count of the box the baseline runs on."""
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return "%s, %d logical CPUs" % (model, os.cpu_count() or 0)


def cpu_baseline_decode(D, Skv, B, H, dtype):
    from oracle import oracle as O
    q, k, v = make_inputs(SEED0 + 3, B, H, H, 1, Skv, D, dtype)
    q, k, v = (dtypes.round_to(x, dtype) for x in (q, k, v))
    t0 = time.perf_counter()
    O.sdpa_materialised(q, k, v)
    dt = time.perf_counter() - t0
    return 2.0 * B * H * Skv * D * 2 / dt / 1e9, dt


def prefill_chunk_leg(steps, warmup, only_shape=None):
    """A chunk of a long prompt: few query rows (one sequence, 128 or 512 new positions) over a long cache, causal.  The
    launch has 32 or 128 (head, row block) items for 256 compute units, so the library splits the key axis and combines
    the partial results; beside it the same launch unsplit (num_splits = 1)."""
    out = {}
    for i, (dt, Sq, Skv) in enumerate(((capi.BF16, 128, 32768), (capi.BF16, 512, 32768), (capi.F32, 128, 32768))):
        B, Hq, Hkv, D = 1, 32, 8, 128
        if only_shape is not None and only_shape != "%s_sq%d_kv%d" % (dtypes.NAMES[dt], Sq, Skv):
            continue
        flops = 4.0 * D * Hq * B * (Sq * Skv - Sq * (Sq - 1) / 2.0)
        peak = PEAK_F32_TFLOPS if dt == capi.F32 else PEAK_BF16_TFLOPS
        kernel = "sdpa_prefill_f32_kernel<128>" if dt == capi.F32 else "sdpa_prefill_mfma_kernel<bf16,128>"
        entry = {"workload": "%s causal prefill chunk B=%d Hq=%d Hkv=%d S_q=%d over KV=%d D=128" % (dtypes.NAMES[dt], B, Hq, Hkv, Sq, Skv)}
        for name, ns in (("auto", 0), ("unsplit", 1)):
            w = Workload("chunk", SEED0 + 60 + i, B, Hq, Hkv, Sq, Skv, D, dt, True, num_splits=ns)
            wall, ev_mean, ev_med, ev_min = w.time(max(steps, 100) if dt != capi.F32 else 20, warmup if dt != capi.F32 else 3)
            ev_mean, ev_from = launch_duration(w, ev_mean)
            entry[name] = {"num_splits": w.splits, "ms_per_step": wall, "tflops": flops / (wall * 1e-3) / 1e12,
                           "roofline": {"bound": "mfma", "achieved": flops / (ev_mean * 1e-3) / 1e12, "peak": peak, "unit": "TFLOP/s",
                                        "frac": flops / (ev_mean * 1e-3) / 1e12 / peak,
                                        "traffic": traffic_of("prefill_chunk/%s_sq%d_kv%d/%s" % (dtypes.NAMES[dt], Sq, Skv, name))[0], "traffic_source": TRAFFIC_PROFILE,
                                        "kernel": kernel + (" over splits of the keys + sdpa_combine_kernel" if w.splits > 1 else ""),
                                        "algorithmic_flops_per_launch": flops, "launch_ms_mean": ev_mean, "launch_ms_mean_from": ev_from, "launch_ms_min": ev_min},
                           "parity_max_abs_err": w.parity(16)}
            w.free()
        out["%s_sq%d_kv%d" % (dtypes.NAMES[dt], Sq, Skv)] = entry
    return out


def decode_gqa_leg(steps, warmup, only_shape=None):
    """Decode shapes beyond BASELINE config 4, where several query rows share a KV head: grouped-query decode at config
    4's batch and cache length, one long sequence, and a short run of query positions (causal among themselves).  Each
    through the kernel AUTO picks (the matrix-core split-KV kernel) and, where it takes the shape, through the
    vector-ALU split-KV kernel; KV bytes read once / launch time against the HBM peak."""
    out = {}
    BF, F = capi.BF16, capi.F32
    shapes = [("gqa4_b32_kv8192", 32, 32, 8, 1, 8192, False, BF), ("gqa4_b1_kv131072", 1, 32, 8, 1, 131072, False, BF),
              ("gqa8_b32_kv8192", 32, 64, 8, 1, 8192, False, BF), ("gqa4_sq4_b8_kv8192", 8, 32, 8, 4, 8192, True, BF),
              # f32 caches (the reference's own dtype): 4 rows per KV head, and 32 (8 heads x 4 positions), where the IEEE-f32
              # matrix instructions - half a PFLOP/s short of the 16-bit ones - come close to being the bound
              ("f32_gqa4_b32_kv8192", 32, 32, 8, 1, 8192, False, F), ("f32_gqa8_sq4_b8_kv8192", 8, 64, 8, 4, 8192, True, F)]
    names = {capi.IMPL_SPLITKV: "sdpa_decode_split_kernel (vector ALU)", capi.IMPL_SPLITKV_MFMA: "sdpa_decode_mfma_kernel (matrix cores)",
             capi.IMPL_MFMA: "sdpa_prefill_mfma_kernel"}
    names_f32 = {capi.IMPL_SPLITKV: "sdpa_decode_split_kernel (vector ALU)", capi.IMPL_SPLITKV_MFMA: "sdpa_decode_f32_kernel (matrix cores, IEEE f32)",
                 capi.IMPL_MFMA: "sdpa_prefill_f32_kernel"}
    for i, (name, B, Hq, Hkv, Sq, Skv, causal, dt) in enumerate(shapes):
        if only_shape is not None and name != only_shape:
            continue
        kv_bytes = 2.0 * B * Hkv * Skv * 128 * (4 if dt == F else 2)
        n = max(steps, min(200, int(0.02 / (kv_bytes / 6e12))))
        entry = {"workload": "%s decode B=%d Hq=%d Hkv=%d S_q=%d KV=%d D=128%s" % (dtypes.NAMES[dt], B, Hq, Hkv, Sq, Skv, " causal" if causal else "")}
        w = Workload("decode_" + name, SEED0 + 40 + i, B, Hq, Hkv, Sq, Skv, 128, dt, causal)
        entry["kv_copies_in_rotation"] = w.rotate_kv()
        for impl in (capi.IMPL_AUTO, capi.IMPL_SPLITKV):
            if impl == capi.IMPL_SPLITKV and (Hq // Hkv) * Sq > 8:
                continue
            if impl != capi.IMPL_AUTO:
                w.replan(impl=impl)
            wall, ev_mean, ev_med, ev_min = w.time(n, warmup)
            ev_mean, ev_from = launch_duration(w, ev_mean)
            entry["auto" if impl == capi.IMPL_AUTO else "vector_alu_kernel"] = {
                "kernel": (names_f32 if dt == F else names).get(w.impl, str(w.impl)), "num_splits": w.splits, "ms_per_step": wall,
                "kv_gb_per_s": kv_bytes / (wall * 1e-3) / 1e9,
                "roofline": {"bound": "hbm", "achieved": kv_bytes / (ev_mean * 1e-3) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                             "frac": kv_bytes / (ev_mean * 1e-3) / 1e9 / PEAK_HBM_GBS,
                             "traffic": traffic_of("decode_gqa/%s/%s" % (name, "auto" if impl == capi.IMPL_AUTO else "vector_alu"))[0], "traffic_source": TRAFFIC_PROFILE,
                             "algorithmic_bytes_per_launch": kv_bytes, "launch_ms_mean": ev_mean, "launch_ms_mean_from": ev_from, "launch_ms_min": ev_min},
                "parity_max_abs_err": w.parity(16)}
        if name == "gqa4_b32_kv8192" and only_shape is None:
            # the same launch with an additive position bias per query head, handed over as the reference's operator takes it: a
            # [1, Hq, 1, KV] mask tensor.  The matrix-core split-KV kernel copies the mask's values into LDS a block ahead.
            bias = (-0.02 * np.arange(Skv)[::-1].astype(np.float32))[None, None, None, :] * (1.0 + np.arange(Hq, dtype=np.float32))[None, :, None, None]
            tm = capi.DeviceBuffer.from_numpy(dtypes.encode(np.ascontiguousarray(bias), dt))
            w.desc.add_mask = tm.ptr
            for a, st in enumerate((0, Skv, 0, 1)):
                w.desc.mask_stride[a] = st
            w.replan()
            wall_b, ev_b, _, _ = w.time(n, warmup)
            ev_b = launch_duration(w, ev_b)[0]
            from oracle import oracle as O
            q, k, v = (dtypes.round_to(x, dt) for x in w.host)
            rows = np.array([[0, 0], [B * Hq - 1, 0], [5, 0], [B * Hq // 2, 0]])
            ref = O.sdpa_rows(q.reshape(B, Hkv, Hq // Hkv, Sq, 128), k[:, :, None], v[:, :, None], rows,
                              mask=dtypes.round_to(bias, dt).reshape(1, Hkv, Hq // Hkv, 1, Skv))
            err = float(np.abs(w.to.to_f32().reshape(B * Hq, Sq, 128)[rows[:, 0], rows[:, 1]] - ref).max())
            entry["with_bias_mask_tensor"] = {"kernel": names.get(w.impl, str(w.impl)), "num_splits": w.splits, "ms_per_step": wall_b,
                                              "kv_gb_per_s": kv_bytes / (wall_b * 1e-3) / 1e9, "frac": kv_bytes / (ev_b * 1e-3) / 1e9 / PEAK_HBM_GBS,
                                              "traffic": traffic_of("decode_gqa/%s/bias" % name)[0], "traffic_source": TRAFFIC_PROFILE,
                                              "parity_max_abs_err": err}
            tm.free()
        w.free()
        out[name] = entry
    return out


def head_dims_leg(steps, warmup, only_shape=None):
    """Head dimensions other than 64 and 128 (bf16): D = 96 runs zero-padded in the 128 instances of the prefill and split-KV
    kernels, D = 256 in the prefill kernel for 256 and in the 256 instance of the split-KV kernel (decode, and a 256-row chunk of a
    16384-token prompt: too few 128-row blocks for the prefill kernel, which does not split the keys).  Prefill: useful FLOPs (4 D per visible
    pair) against the bf16 matrix peak; decode: KV bytes read once against the HBM peak."""
    out = {}
    names = {capi.IMPL_SPLITKV_MFMA: "sdpa_decode_mfma_kernel", capi.IMPL_MFMA: "sdpa_prefill_mfma_kernel", capi.IMPL_GENERIC: "sdpa_generic_kernel"}
    for i, (name, B, Hq, Hkv, Sq, Skv, D, causal) in enumerate((("prefill_d96", 8, 16, 16, 2048, 2048, 96, True), ("prefill_d256", 4, 16, 16, 4096, 4096, 256, True),
                                                                 ("chunk_d256", 1, 32, 8, 256, 16384, 256, True),
                                                                 ("decode_d96", 32, 32, 8, 1, 8192, 96, False), ("decode_d256", 32, 32, 8, 1, 8192, 256, False),
                                                                 ("prefill_d96_s4096", 8, 16, 16, 4096, 4096, 96, True))):      # (config 3's shape at D = 96)
        if only_shape is not None and name != only_shape:
            continue
        w = Workload("head_dims_" + name, SEED0 + 80 + i, B, Hq, Hkv, Sq, Skv, D, capi.BF16, causal)
        copies = w.rotate_kv() if Sq == 1 else 1
        wall, ev_mean, ev_med, ev_min = w.time(max(steps, 50), warmup)
        ev_mean, ev_from = launch_duration(w, ev_mean)
        entry = {"workload": "bf16 %s B=%d Hq=%d Hkv=%d S_q=%d KV=%d D=%d" % ("decode" if Sq == 1 else "causal prefill" if Sq == Skv else "causal prefill chunk", B, Hq, Hkv, Sq, Skv, D),
                 "kernel": "sdpa_prefill_wide_kernel" if D > 128 and w.impl == capi.IMPL_MFMA else names.get(w.impl, str(w.impl)),
                 "num_splits": w.splits, "ms_per_step": wall, "parity_max_abs_err": w.parity(16)}
        if Sq == 1:
            entry["kv_copies_in_rotation"] = copies
        if Sq > 1:
            flops = causal_flops(B, Hq, Sq, Skv, D)
            entry["tflops"] = flops / (wall * 1e-3) / 1e12
            entry["roofline"] = {"bound": "mfma", "achieved": flops / (ev_mean * 1e-3) / 1e12, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                                 "frac": flops / (ev_mean * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
                                 "traffic": traffic_of("head_dims/" + name)[0], "traffic_source": TRAFFIC_PROFILE,
                                 "algorithmic_flops_per_launch": flops, "launch_ms_mean": ev_mean, "launch_ms_mean_from": ev_from, "launch_ms_min": ev_min}
        else:
            kv_bytes = 2.0 * B * Hkv * Skv * D * 2
            entry["kv_gb_per_s"] = kv_bytes / (wall * 1e-3) / 1e9
            entry["roofline"] = {"bound": "hbm", "achieved": kv_bytes / (ev_mean * 1e-3) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                 "frac": kv_bytes / (ev_mean * 1e-3) / 1e9 / PEAK_HBM_GBS,
                                 "traffic": traffic_of("head_dims/" + name)[0], "traffic_source": TRAFFIC_PROFILE,
                                 "algorithmic_bytes_per_launch": kv_bytes, "launch_ms_mean": ev_mean, "launch_ms_mean_from": ev_from, "launch_ms_min": ev_min}
        w.free()
        out[name] = entry
    return out


def decode_step_graph(w, B, H, Skv, D, steps):
    """One decode step as a serving loop runs it: append the token's K and V rows to the cache at kv_lens (device side),
    attend over the cache with kv_lens; both recorded into a launch graph once and replayed per token."""
    lens = capi.DeviceBuffer.from_numpy(np.full(B, Skv - 1, np.int32))       # one free row: every step sees all Skv keys
    kn, vn = (host.DeviceTensor((B, H, 1, D), capi.BF16) for _ in range(2))
    ad = capi.KvAppendDesc()
    ad.dtype, ad.device = capi.BF16, 0
    ad.B, ad.Hkv, ad.S_new, ad.S_max, ad.D, ad.Dv = B, H, 1, Skv, D, D
    ad.k_new, ad.v_new, ad.k_cache, ad.v_cache, ad.kv_lens = kn.ptr, vn.ptr, w.tk.ptr, w.tv.ptr, lens.ptr
    for name, S in (("k_new_stride", 1), ("v_new_stride", 1), ("k_cache_stride", Skv), ("v_cache_stride", Skv)):
        st = getattr(ad, name)
        st[0], st[1], st[2] = H * S * D, S * D, D
    w.desc.kv_lens = lens.ptr
    stream = capi.Stream()
    with capi.Graph.record(stream) as graph:
        capi.kv_append(ad, stream.ptr)
        capi.sdpa_fwd(w.desc, stream.ptr)
    for _ in range(10):
        graph.launch()
    stream.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        graph.launch()
    stream.sync()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    graph.destroy()
    stream.destroy()
    w.desc.kv_lens = None
    for t in (lens, kn.buf, vn.buf):
        t.free()
    return {"what": "kv_append (1 token) + attention over the cache with device-side kv_lens, one graph replay per step",
            "ms_per_step": ms, "kv_GBps": 2.0 * B * H * Skv * D * 2 / (ms * 1e-3) / 1e9}


def backward_leg(steps, warmup, dtype=capi.BF16, B=8, H=16, S=4096, D=128, what="BASELINE config 3's shape"):
    """Forward (keeping the row normalisers) and then the timed backward: dQ, dK, dV for a synthetic upstream gradient.
    The figure counts 2.5 x the forward's FLOPs (five matrix products against the forward's two; the recomputation of S
    and dP in both big kernels is not counted)."""
    name = {capi.BF16: "bf16", capi.F16: "f16", capi.F32: "f32"}[dtype]
    q, k, v = make_inputs(SEED0 + 5, B, H, H, S, S, D, dtype)
    g = rng(SEED0 + 6).standard_normal((B, H, S, D), dtype=np.float32)
    tq, tk, tv, tg = (host.DeviceTensor.from_f32(x, dtype) for x in (q, k, v, g))
    to, tdq, tdk, tdv = (host.DeviceTensor((B, H, S, D), dtype) for _ in range(4))
    lse = capi.DeviceBuffer(B * H * S * 4)
    bd = capi.SdpaBwdDesc()
    bd.fwd = host.make_desc(tq, tk, tv, to, causal=True, lse=lse)
    capi.sdpa_fwd(bd.fwd)
    for field, t in (("d_o", tg), ("d_q", tdq), ("d_k", tdk), ("d_v", tdv)):
        setattr(bd, field, t.ptr)
        st = host._strides3(t.shape)
        for i in range(3):
            getattr(bd, field + "_stride")[i] = st[i]
    ws = capi.DeviceBuffer(capi.sdpa_bwd_workspace(bd))
    bd.workspace, bd.workspace_bytes = ws.ptr, ws.nbytes
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < 0.15:          # clocks settle (set-up, not measurement)
        capi.sdpa_bwd(bd)
        capi.sync()
    for _ in range(warmup):
        capi.sdpa_bwd(bd)
    capi.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        capi.sdpa_bwd(bd)
    capi.sync()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    # at-size check of one (batch, head) slice against the float64 backward oracle (checker only)
    from oracle import sdpa_backward as OB
    b, h = B - 1, H - 1
    rq, rk, rv, rg = (dtypes.round_to(x[b, h], dtype) for x in (q, k, v, g))
    ref = OB.sdpa_backward(rq, rk, rv, rg, causal=True)
    err = max(float(np.abs(t.to_f32()[b, h] - r).max() / np.abs(r).max()) for t, r in zip((tdq, tdk, tdv), ref))
    flops = 2.5 * causal_flops(B, H, S, S, D)
    for t in (tq.buf, tk.buf, tv.buf, tg.buf, to.buf, tdq.buf, tdk.buf, tdv.buf, lse, ws):
        t.free()
    peak = PEAK_F32_TFLOPS if dtype == capi.F32 else PEAK_BF16_TFLOPS
    return {"workload": "backward of %s: %s causal B=%d H=%d S=%d D=%d, dQ dK dV from Q K V O dO and the "
                        "forward's row normalisers" % (what, name, B, H, S, D),
            "step": "one incin_rocm_sdpa_bwd call (3 kernels: row dots, dQ, dK/dV)", "dtype": name,
            "metric": "attn bwd TFLOP/s (2.5 x forward FLOPs)", "value": flops / (wall * 1e-3) / 1e12, "unit": "TFLOP/s",
            "ms_per_step": wall, "steps": steps, "frac_of_%s_mfma_peak" % ("fp32" if dtype == capi.F32 else "bf16"): flops / (wall * 1e-3) / 1e12 / peak,
            "traffic": traffic_of("backward/%s_d%d" % (name, D))[0], "traffic_source": TRAFFIC_PROFILE,
            "parity_max_err_rel_to_max_abs_ref": err,
            "parity_sample": "dQ, dK, dV of slice (b=%d, h=%d) against the float64 oracle of the reference's tape gradients" % (b, h)}


def read_rate():
    """What the memory system delivers to a kernel that only reads (incin_rocm_read_rate: 16-byte loads of 4 GiB, 8 in
    flight per lane, summed and thrown away), with non-temporal loads and with plain ones - the measured ceiling the
    split-KV kernels live under, reported beside the nominal HBM figure their roofline is priced against."""
    nbytes = 4 << 30
    src = capi.DeviceBuffer(nbytes)
    capi.check(capi.load().incin_rocm_memset(0, src.ptr, 0x11, nbytes))
    sink = capi.DeviceBuffer(16384)
    out = {"what": "rate of a read-only kernel over 4 GiB (16-byte loads, 4096 workgroups of 256 threads, 8 loads in flight per lane)",
           "unit": "GB/s", "nominal_peak": PEAK_HBM_GBS}
    for name, nt in (("non_temporal_loads", True), ("plain_loads", False)):
        for _ in range(5):
            capi.read_rate(src, nbytes, nt, sink)
        capi.sync()
        best = None
        for _ in range(3):
            e0, e1 = capi.Event(), capi.Event()
            e0.record()
            for _ in range(10):
                capi.read_rate(src, nbytes, nt, sink)
            e1.record()
            capi.sync()
            ms = e0.elapsed_ms(e1) / 10
            best = ms if best is None else min(best, ms)
            e0.destroy(); e1.destroy()
        out[name] = {"value": nbytes / (best * 1e-3) / 1e9, "ms": best, "frac_of_nominal": nbytes / (best * 1e-3) / 1e9 / PEAK_HBM_GBS}
    src.free()
    sink.free()
    return out


def matrix_rate():
    """What rate of bf16 matrix instructions the device sustains, by the data they work on: a loop of
    v_mfma_f32_32x32x16_bf16 on every compute unit (incin_rocm_matrix_rate), about 20 ms per launch, on zeros, on N(0,1)
    values rounded to bf16 (what the attention inputs are) and with the vector / LDS instructions the prefill kernel issues
    per matrix instruction.  The device lowers its clock under the switching activity of real data; these figures are the
    ceilings the 16-bit attention kernels live under, reported beside the nominal peak the roofline is priced against."""
    out = {"what": "sustained rate of a loop of v_mfma_f32_32x32x16_bf16, 2 wavefronts per SIMD on every CU, ~20 ms launches; "
                   "operands: 256 KiB of zeros or of N(0,1) rounded to bf16; mix 1 adds, per matrix instruction, 2 v_exp_f32, "
                   "3 v_fma_f32 and one ds_read_b128", "unit": "TFLOP/s", "nominal_peak": PEAK_BF16_TFLOPS}
    sink = capi.DeviceBuffer(2048 * 1024)
    data = {"zeros": np.zeros(65536, np.uint32),
            "normal": dtypes.f32_to_bf16_bits(rng(SEED0 + 9).standard_normal(131072, dtype=np.float32)).view(np.uint32)}
    for name, arr in data.items():
        src = capi.DeviceBuffer.from_numpy(arr)
        for mix in (0, 1):
            iters = 150000 if mix == 0 else 100000
            capi.matrix_rate(src, sink, mix, 2000)
            capi.sync()
            best = None
            for _ in range(3):
                e0, e1 = capi.Event(), capi.Event()
                e0.record()
                fl = capi.matrix_rate(src, sink, mix, iters)
                e1.record()
                capi.sync()
                ms = e0.elapsed_ms(e1)
                best = ms if best is None else min(best, ms)
                e0.destroy(); e1.destroy()
            out["%s_operands_mix%d" % (name, mix)] = {"value": fl / (best * 1e-3) / 1e12, "ms": best,
                                                       "frac_of_nominal": fl / (best * 1e-3) / 1e12 / PEAK_BF16_TFLOPS}
        src.free()
    sink.free()
    # the attention kernel itself, same launch (configuration 3), by what its inputs hold: N(0,1) (the headline figure),
    # the same values scaled by 0.01 (near-uniform probabilities) and zeros - identical instruction stream and traffic
    B, H, S, D = 8, 16, 4096, 128
    flops = causal_flops(B, H, S, S, D)
    r = rng(SEED0 + 10)
    x = r.standard_normal((B, H, S, D), dtype=np.float32)
    by_data = {}
    for name, scale in (("normal", 1.0), ("normal_times_0.01", 0.01), ("zeros", 0.0)):
        tq, tk, tv = (host.DeviceTensor.from_f32(np.roll(x, sh, axis=2) * np.float32(scale), capi.BF16) for sh in (0, 1, 2))
        to = host.DeviceTensor((B, H, S, D), capi.BF16)
        d = host.make_desc(tq, tk, tv, to, causal=True)
        for _ in range(120):
            capi.sdpa_fwd(d)
        capi.sync()
        e0, e1 = capi.Event(), capi.Event()
        e0.record()
        for _ in range(60):
            capi.sdpa_fwd(d)
        e1.record()
        capi.sync()
        ms = e0.elapsed_ms(e1) / 60
        e0.destroy(); e1.destroy()
        by_data[name] = {"ms_per_launch": ms, "value": flops / (ms * 1e-3) / 1e12}
        for t in (tq, tk, tv, to):
            t.buf.free()
    out["prefill_config3_by_input_data"] = by_data
    return out


def f32_configs(steps, warmup, with_cpu, threads):
    """BASELINE configs 1 and 2 - f32, the one dtype the reference's operator runs end to end - on the IEEE-f32
    matrix-core kernel: absolute TFLOP/s against the fp32 matrix peak, config 2 also with the causal mask handed over
    as the explicit [S, S] tensor of 0 / -inf a caller of the reference's operator passes, and the oracle's
    materialising restatement timed on all of config 2 beside it."""
    from oracle import oracle as O
    out = {}
    for key, (B, H, S, D, causal, scale_note) in (("f32_c1", (1, 1, 128, 64, False, "scale=0.125")),
                                                  ("f32_c2", (4, 8, 1024, 64, True, "scale=1/sqrt(64)")),
                                                  ("f32_large", (8, 16, 4096, 128, True, "scale=1/sqrt(128)"))):
        w = Workload(key, SEED0 + {"f32_c1": 0, "f32_c2": 1, "f32_large": 7}[key], B, H, H, S, S, D, capi.F32, causal)
        n = max(steps, 200) if key != "f32_large" else max(5, min(steps, 20))      # launches of tens of microseconds / of ~5 ms
        wall, ev_mean, ev_med, ev_min = w.time(n, warmup)
        flops = causal_flops(B, H, S, S, D) if causal else 4.0 * D * B * H * S * S
        dur, dur_from = launch_duration(w, ev_mean)
        kernel = {capi.IMPL_MFMA: "sdpa_prefill_f32_kernel<%d>" % D, capi.IMPL_GENERIC: "sdpa_generic_kernel<float>",
                  capi.IMPL_SPLITKV_MFMA: "sdpa_decode_f32_kernel<%d> (the f32 split-KV kernel, 32 rows per workgroup: AUTO's choice for launches "
                                          "of at most one 128-row block per compute unit)" % D}.get(w.impl, str(w.impl))
        what = "BASELINE config %s" % key[-1] if key != "f32_large" else "not a BASELINE config (the shape of config 3 in f32: a launch that fills the machine)"
        rec = {"workload": "%s: f32 %s attention fwd B=%d H=%d S_q=S_kv=%d D=%d, %s" %
                           (what, "causal" if causal else "non-causal", B, H, S, D, scale_note),
               "metric": "attn fwd TFLOP/s", "value": flops / (wall * 1e-3) / 1e12, "unit": "TFLOP/s", "dtype": "f32",
               "ms_per_step": wall, "steps": n,
               "roofline": {"bound": "mfma", "achieved": flops / (dur * 1e-3) / 1e12, "peak": PEAK_F32_TFLOPS, "unit": "TFLOP/s",
                            "frac": flops / (dur * 1e-3) / 1e12 / PEAK_F32_TFLOPS,
                            "traffic": traffic_of("f32/" + key)[0], "traffic_source": TRAFFIC_PROFILE, "kernel": kernel,
                            "algorithmic_flops_per_launch": flops, "launch_ms_mean": dur, "launch_ms_mean_from": dur_from,
                            "launch_ms_event_pair_mean": ev_mean, "launch_ms_median": ev_med, "launch_ms_min": ev_min},
               "parity_max_abs_err": w.parity()}
        if w.impl != capi.IMPL_MFMA:        # the f32 prefill kernel on the same launch, pinned
            w.replan(impl=capi.IMPL_MFMA)
            wall_p = w.time(n, warmup)[0]
            rec["prefill_kernel_pinned"] = {"kernel": "sdpa_prefill_f32_kernel<%d>" % D, "ms_per_step": wall_p,
                                            "value": flops / (wall_p * 1e-3) / 1e12, "unit": "TFLOP/s", "parity_max_abs_err": w.parity()}
            w.replan()
        if key == "f32_c2":
            # the same problem with the mask as a tensor: the launch first classifies the tensor by blocks of 32 x 32 (hidden
            # blocks are skipped, zero blocks run unmasked), FLOPs counted as above
            mask = O.causal_additive_mask(S, S)
            tm = capi.DeviceBuffer.from_numpy(mask)
            w.desc.causal = 0
            w.desc.add_mask = tm.ptr
            for i, st in enumerate((0, 0, S, 1)):
                w.desc.mask_stride[i] = st
            mbytes = capi.sdpa_workspace(w.desc)[0]            # block flags of the mask
            mws = capi.DeviceBuffer(mbytes) if mbytes else None
            if mws is not None:
                w.desc.workspace, w.desc.workspace_bytes = mws.ptr, mws.nbytes
            wall_m = w.time(n, warmup)[0]
            rec["with_dense_mask_tensor"] = {"what": "causal mask passed as an f32 [S, S] additive tensor (add_mask) instead of the causal flag",
                                             "ms_per_step": wall_m, "value": flops / (wall_m * 1e-3) / 1e12, "unit": "TFLOP/s",
                                             "parity_max_abs_err": w.parity()}
            tm.free()
            if mws is not None:
                mws.free()
            if with_cpu:
                q, k, v = w.host
                t0 = time.perf_counter()
                O.sdpa_materialised(q, k, v, mask=mask)
                dt = time.perf_counter() - t0
                rec["cpu_baseline"] = {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
                                       "sample": "all of config 2 (32 (b,h) slices, explicit 0/-inf causal mask), oracle's materialising "
                                                 "restatement of the reference CPU op (not the Rust binary); %.1f s; host: %s" % (dt, host_cpu())}
        w.free()
        out[key] = rec
    return out


def _round(x, sig=6):
    """Floats to `sig` significant digits, recursively: the compact line carries figures, not 17-digit reprs."""
    if isinstance(x, float):
        return float("%.*g" % (sig, x))
    if isinstance(x, dict):
        return {k: _round(v, sig) for k, v in x.items()}
    if isinstance(x, (list, tuple)):
        return [_round(v, sig) for v in x]
    return x


def _pick(d, keys):
    return {k: d[k] for k in keys if d is not None and k in d}


_ROOFLINE_KEYS = ("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel", "algorithmic_flops_per_launch",
                  "algorithmic_bytes_per_launch", "launch_ms_mean", "launch_ms_median", "launch_ms_min")
COMPACT_LIMIT = 4096


def compact_line(result, detail_file="bench_detail.json"):
    """The one line a harness parses: the headline (config 3) with its roofline and CPU baseline, config 4's decode and
    config 5's ragged prefill in short form.  Everything else the run measured stays in `detail_file`."""
    out = _pick(result, ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                         "vs_baseline", "dtype", "data", "config"))
    if "roofline" in result:
        out["roofline"] = _pick(result["roofline"], _ROOFLINE_KEYS)
    if "cpu_baseline" in result:
        out["cpu_baseline"] = _pick(result["cpu_baseline"], ("value", "unit", "cores", "kind", "sample"))
    if "parity_max_abs_err" in result:
        out["parity_max_abs_err"] = result["parity_max_abs_err"]
    dec = result.get("decode")
    if dec:
        d = _pick(dec, ("workload", "value", "unit", "ms_per_step", "parity_max_abs_err"))
        d["roofline"] = _pick(dec.get("roofline"), _ROOFLINE_KEYS)
        if "cpu_baseline" in dec:
            d["cpu_baseline"] = _pick(dec["cpu_baseline"], ("value", "unit", "cores", "kind", "sample"))
        out["decode"] = d
    pl = result.get("prefill_long")
    if pl:
        d = _pick(pl, ("value", "unit", "ms_per_step", "parity_max_abs_err"))
        d["roofline"] = _pick(pl.get("roofline"), ("frac", "launch_ms_mean"))
        out["prefill_long"] = d
    bw = result.get("backward")
    if bw:
        out["backward"] = _pick(bw, ("value", "unit", "ms_per_step", "frac_of_bf16_mfma_peak"))
    out["detail"] = detail_file
    line = json.dumps(_round(out), separators=(",", ":"))
    if len(line) >= COMPACT_LIMIT:      # never let free text push the line past what a tail-reading harness keeps
        for obj in (out.get("cpu_baseline"), out.get("decode", {}).get("cpu_baseline")):
            if obj and "sample" in obj:
                obj["sample"] = obj["sample"][:160]
        line = json.dumps(_round(out), separators=(",", ":"))
    assert len(line) < COMPACT_LIMIT, "compact bench line is %d bytes" % len(line)
    return line


_T0 = time.perf_counter()


def note(leg):
    """Progress on stderr (stdout carries the one JSON line): a run that prints nothing for minutes looks hung to a harness."""
    print("[bench %6.1f s] %s" % (time.perf_counter() - _T0, leg), file=sys.stderr, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--with-mask-tensor", action="store_true", help="with --only prefill: also the launch with the causal mask as a tensor (for profiles)")
    ap.add_argument("--no-padding-compare", action="store_true",
                    help="prefill_long: skip the extra timing of the batch with its padding rows computed (profiling: every "
                         "launch of the run is then the same launch)")
    ap.add_argument("--shape", "--decode-gqa-shape", dest="shape", default=None,
                    help="with --only decode_gqa, head_dims or prefill_chunk: one of the leg's shapes by name (for profiles)")
    ap.add_argument("--only", choices=["prefill", "prefill_long", "prefill_chunk", "decode", "decode_gqa", "head_dims", "backward", "f32", "copy", "matrix_rate", "read_rate"], default=None,
                    help="run a single workload (profiling). 'copy' runs --steps device-to-device copies of 1 GiB "
                         "through the library's plain copy kernel: the known-size dispatch that hardware byte "
                         "counters (FETCH_SIZE / WRITE_SIZE) are calibrated against")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path shards over batch and kv-head groups "
              "with no communication; no multi-GPU figure is produced). Re-run with --gpus 1.", file=sys.stderr)
        return 2

    capi.load()
    info = capi.device_info(0)
    try:
        ncores = len(os.sched_getaffinity(0))
    except AttributeError:
        ncores = os.cpu_count()
    threads = int(os.environ.get("OMP_NUM_THREADS", ncores))

    result = {
        "metric": METRIC, "value": None, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": None, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic: Q,K,V i.i.d. N(0,1) from numpy PCG64(seed 20261125+config), rounded to bf16",
        "config": {"workload": "BASELINE config 3: bf16 causal prefill B=8 H=16 S_q=S_kv=4096 D=128, scale=1/sqrt(128), "
                               "f32 accumulate, bf16 out", "step": "one incin_rocm_sdpa_fwd launch"},
        "device": {"name": info.name.decode() or info.arch.decode().split(":")[0], "arch": info.arch.decode(),
                   "compute_units": info.compute_units, "clock_khz": info.clock_khz},
    }

    if args.only == "copy":
        n = 1 << 30
        a, b = capi.DeviceBuffer(n), capi.DeviceBuffer(n)
        capi.check(capi.load().incin_rocm_memset(0, a.ptr, 1, n))
        t0 = time.perf_counter()
        for _ in range(args.steps):
            capi.check(capi.load().incin_rocm_memcpy_d2d(0, b.ptr, a.ptr, n))
        dt = (time.perf_counter() - t0) / args.steps
        print(json.dumps({"metric": "copy16_kernel 1 GiB device-to-device", "bytes_read": n, "bytes_written": n,
                          "ms_per_copy": dt * 1e3, "GBps_read_plus_write": 2 * n / dt / 1e9}))
        return 0

    if args.only in (None, "prefill"):
        note("prefill")
        B, H, S, D = 8, 16, 4096, 128
        w = Workload("prefill_c3", SEED0 + 2, B, H, H, S, S, D, capi.BF16, True)
        wall, ev_mean, ev_med, ev_min = w.time(args.steps, args.warmup)
        flops = causal_flops(B, H, S, S, D)
        result["value"] = flops / (wall * 1e-3) / 1e12
        result["ms_per_step"] = wall
        result["roofline"] = {"bound": "mfma", "achieved": flops / (ev_mean * 1e-3) / 1e12, "peak": PEAK_BF16_TFLOPS,
                              "unit": "TFLOP/s", "frac": flops / (ev_mean * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, "traffic": traffic_of("prefill")[0],
                              "traffic_source": traffic_of("prefill")[1], "kernel": "sdpa_prefill_mfma_kernel<bf16,128>", "algorithmic_flops_per_launch": flops,
                              "launch_ms_mean": ev_mean, "launch_ms_median": ev_med, "launch_ms_min": ev_min}
        result["parity_max_abs_err"] = w.parity()
        if args.only is None or args.with_mask_tensor:
            # the same batch with the causal mask handed over the way the reference's operator takes it: an explicit
            # [S, S] tensor of 0 / -inf (bf16, broadcast over batch and heads) instead of the causal flag
            from oracle import oracle as O
            tm = capi.DeviceBuffer.from_numpy(dtypes.encode(O.causal_additive_mask(S, S), capi.BF16))
            w.desc.causal = 0
            w.desc.add_mask = tm.ptr
            for i, st in enumerate((0, 0, S, 1)):
                w.desc.mask_stride[i] = st
            mws = capi.DeviceBuffer(capi.sdpa_workspace(w.desc)[0])
            w.desc.workspace, w.desc.workspace_bytes = mws.ptr, mws.nbytes
            wall_m = w.time(args.steps, args.warmup)[0]
            result["prefill_with_dense_mask_tensor"] = {
                "what": "config 3 with the causal mask passed as a bf16 [S, S] additive tensor (add_mask); the launch classifies it "
                        "by 32 x 32 blocks and takes a limit per mask row first, then runs the blocks whose rows all have a limit "
                        "from the limits; same FLOP count", "ms_per_step": wall_m, "value": flops / (wall_m * 1e-3) / 1e12,
                "unit": "TFLOP/s", "ratio_to_causal_flag": wall / wall_m, "parity_max_abs_err": w.parity()}
            tm.free()
            mws.free()
            # and with a mask that has values: a distance bias under the causal triangle (-0.01 per key of distance, -inf above
            # the diagonal) - no row limit describes it; the kernel takes the values through LDS, a tile ahead
            dist = np.arange(S, dtype=np.float32)[:, None] - np.arange(S, dtype=np.float32)[None, :]
            bias = np.where(dist >= 0, -0.01 * dist, -np.inf).astype(np.float32)
            tm = capi.DeviceBuffer.from_numpy(dtypes.encode(bias, capi.BF16))
            w.desc.add_mask = tm.ptr
            w.desc.workspace, w.desc.workspace_bytes = None, 0
            mws = capi.DeviceBuffer(capi.sdpa_workspace(w.desc)[0])
            w.desc.workspace, w.desc.workspace_bytes = mws.ptr, mws.nbytes
            wall_b = w.time(args.steps, args.warmup)[0]
            # (parity on sampled rows, against the oracle given the same tensor: the workload's own check knows the causal flag only)
            qh, kh, vh = (dtypes.round_to(x, capi.BF16) for x in w.host)
            rr = rng(98)
            rows = np.stack([rr.integers(0, B * H, 48), rr.integers(0, S, 48)], axis=1)
            rows[0], rows[1] = (0, 0), (B * H - 1, S - 1)
            ref = O.sdpa_rows(qh.reshape(B, H, 1, S, D), kh[:, :, None], vh[:, :, None], rows, mask=dtypes.round_to(bias, capi.BF16).reshape(1, 1, 1, S, S))
            got = w.to.to_f32().reshape(B * H, S, D)[rows[:, 0], rows[:, 1]]
            result["prefill_with_bias_tensor"] = {
                "what": "config 3 with a distance bias under the causal triangle as a bf16 [S, S] additive tensor (values: no "
                        "row limit describes it); same FLOP count", "ms_per_step": wall_b, "value": flops / (wall_b * 1e-3) / 1e12,
                "unit": "TFLOP/s", "ratio_to_causal_flag": wall / wall_b, "parity_max_abs_err": float(np.abs(got - ref).max()),
                "parity_sample": "48 sampled rows against the oracle given the same tensor"}
            tm.free()
            mws.free()
        w.free()
        if not args.no_cpu_baseline:
            slices = 12
            val, dt = cpu_baseline_prefill(D, S, slices, capi.BF16)
            result["cpu_baseline"] = {
                "value": val, "unit": "TFLOP/s", "cores": threads, "kind": "port",
                "sample": "%d of 128 (b,h) slices of config 3 (S=4096, D=128, explicit 0/-inf causal mask), oracle's "
                          "materialising restatement of the reference CPU op (not the Rust binary): matmuls and "
                          "reductions on 1 thread, elementwise maps on %d OpenMP threads; %.1f s; same causal FLOP count; host: %s"
                          % (slices, threads, dt, host_cpu())}

    if args.only in (None, "prefill_long"):
        note("prefill_long")
        # BASELINE config 5: grouped queries, batch padded to 16384 tokens, causal + key padding; lengths U[2048, 16384]
        # from the same seeded generator
        B, Hq, Hkv, S, D = 4, 32, 8, 16384, 128
        lens = rng(SEED0 + 4).integers(2048, S + 1, B).astype(np.int64)
        w = Workload("prefill_c5", SEED0 + 4, B, Hq, Hkv, S, S, D, capi.BF16, True, kv_lens=lens, pad_queries=True)
        steps = max(5, min(args.steps, 20))                 # ~5 ms per launch
        # first the same batch with the padding rows computed (what a caller gets who can only hand over a key mask)
        wall_all_rows = None
        if not args.no_padding_compare:
            w.desc.q_lens = None
            wall_all_rows = w.time(steps, 2)[0]
            w.desc.q_lens = w.tl.ptr
        wall, ev_mean, ev_med, ev_min = w.time(steps, min(args.warmup, 5))
        flops = 4.0 * D * Hq * float(sum(int(n) * (int(n) + 1) // 2 for n in lens))      # rows i < lens[b] only
        kernel = {capi.IMPL_MFMA: "sdpa_prefill_mfma_kernel<bf16,128>"}.get(w.impl, str(w.impl))
        result["prefill_long"] = {
            "workload": "BASELINE config 5: bf16 GQA causal prefill B=4 Hq=32 Hkv=8 S=16384 (padded) D=128, key padding with "
                        "lengths %s given as kv_lens and q_lens (padding rows not computed); FLOPs count rows and keys inside "
                        "each length only" % lens.tolist(),
            "metric": "attn fwd TFLOP/s", "value": flops / (wall * 1e-3) / 1e12, "unit": "TFLOP/s", "ms_per_step": wall, "steps": steps,
            "roofline": {"bound": "mfma", "achieved": flops / (ev_mean * 1e-3) / 1e12, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                         "frac": flops / (ev_mean * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, "traffic": traffic_of("prefill_long")[0],
                         "traffic_source": traffic_of("prefill_long")[1], "kernel": kernel,
                         "algorithmic_flops_per_launch": flops, "launch_ms_mean": ev_mean, "launch_ms_median": ev_med,
                         "launch_ms_min": ev_min},
            "ms_per_step_with_padding_rows_computed": wall_all_rows,
            "parity_max_abs_err": w.parity(16)}
        w.free()

    if args.only in (None, "decode"):
        note("decode")
        B, H, Skv, D = 32, 32, 8192, 128
        w = Workload("decode_c4", SEED0 + 3, B, H, H, 1, Skv, D, capi.BF16, False)
        wall, ev_mean, ev_med, ev_min = w.time(args.steps, args.warmup)
        kv_bytes = 2.0 * B * H * Skv * D * 2
        dec = {"workload": "BASELINE config 4: bf16 decode MHA B=32 H=32 S_q=1 KV=8192 D=128",
               "metric": "decode KV GB/s", "value": kv_bytes / (wall * 1e-3) / 1e9, "unit": "GB/s", "ms_per_step": wall,
               "num_splits": w.splits,
               "roofline": {"bound": "hbm", "achieved": kv_bytes / (ev_mean * 1e-3) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                            "frac": kv_bytes / (ev_mean * 1e-3) / 1e9 / PEAK_HBM_GBS, "traffic": traffic_of("decode")[0],
                            "traffic_source": traffic_of("decode")[1],
                            "kernel": {capi.IMPL_SPLITKV: "sdpa_decode_split_kernel<bf16,128,1,8> + sdpa_combine_kernel",
                                       capi.IMPL_SPLITKV_MFMA: "sdpa_decode_mfma_kernel<bf16,5,1>"}.get(w.impl, str(w.impl)),
                            "algorithmic_bytes_per_launch": kv_bytes,
                            "launch_ms_mean": ev_mean, "launch_ms_median": ev_med, "launch_ms_min": ev_min},
               "parity_max_abs_err": w.parity()}
        # the same through the vector-ALU split-KV kernel (what one row per KV head over short caches runs on)
        w.replan(impl=capi.IMPL_SPLITKV)
        wall_v, ev_v, _, _ = w.time(args.steps, args.warmup)
        dec["vector_alu_kernel"] = {"kernel": "sdpa_decode_split_kernel<bf16,128,1,8> + sdpa_combine_kernel", "num_splits": w.splits,
                                    "ms_per_step": wall_v, "launch_ms_mean": ev_v, "frac": kv_bytes / (ev_v * 1e-3) / 1e9 / PEAK_HBM_GBS,
                                    "traffic": traffic_of("decode/vector_alu")[0], "traffic_source": TRAFFIC_PROFILE,
                                    "parity_max_abs_err": w.parity()}
        # (last: the appended rows overwrite the end of the cache)
        w.replan()
        dec["decode_step_graph"] = decode_step_graph(w, B, H, Skv, D, args.steps)
        w.free()
        if not args.no_cpu_baseline:
            val, dt = cpu_baseline_decode(D, Skv, 32, 32, capi.BF16)
            dec["cpu_baseline"] = {"value": val, "unit": "GB/s", "cores": threads, "kind": "port",
                                   "sample": "all of config 4 (B=32, H=32, KV=8192, D=128), oracle's materialising restatement of "
                                             "the reference CPU op (serial matmuls and reductions); %.1f s; host: %s" % (dt, host_cpu())}
        result["decode"] = dec

    if args.only in (None, "prefill_chunk"):
        note("prefill_chunk")
        result["prefill_chunk"] = prefill_chunk_leg(args.steps, args.warmup, args.shape)

    if args.only in (None, "decode_gqa"):
        note("decode_gqa")
        result["decode_gqa"] = decode_gqa_leg(args.steps, args.warmup, args.shape)

    if args.only in (None, "head_dims"):
        note("head_dims")
        result["head_dims"] = head_dims_leg(args.steps, args.warmup, args.shape)

    if args.only in (None, "f32"):
        note("f32")
        result.update(f32_configs(args.steps, args.warmup, not args.no_cpu_baseline, threads))

    if args.only in (None, "matrix_rate"):
        note("matrix_rate")
        result["matrix_rate"] = matrix_rate()

    if args.only in (None, "read_rate"):
        note("read_rate")
        result["read_rate"] = read_rate()

    if args.only in (None, "backward"):
        note("backward")
        result["backward"] = backward_leg(max(5, min(args.steps, 30)), min(args.warmup, 5))
        # f32, the dtype the reference trains in: BASELINE config 2's shape (launches of ~100 us) and config 3's
        result["backward_d64"] = backward_leg(max(5, min(args.steps, 30)), min(args.warmup, 5), capi.BF16, 8, 32, 4096, 64, "config 3 with 32 heads of 64 (the same FLOPs)")
        result["backward_f32_c2"] = backward_leg(max(args.steps, 100), min(args.warmup, 5), capi.F32, 4, 8, 1024, 64, "BASELINE config 2's shape")
        result["backward_f32_large"] = backward_leg(max(5, min(args.steps, 10)), min(args.warmup, 3), capi.F32, what="BASELINE config 3's shape in f32")

    for detail in (os.path.join(ROOT, "bench_detail.json"), os.path.join(ROOT, "gpurun_out", "bench_detail.json")):
        if not os.path.isdir(os.path.dirname(detail)):
            continue
        try:
            with open(detail, "w") as f:
                json.dump(result, f, indent=1)
        except OSError as e:                 # a read-only tree must not cost the run its headline
            print("bench.py: could not write %s: %s" % (detail, e), file=sys.stderr)
    print(json.dumps(result), file=sys.stderr, flush=True)
    print(compact_line(result), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
