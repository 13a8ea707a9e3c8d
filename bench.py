#!/usr/bin/env python3
"""Benchmark of the gfx950 blit engine on one MI355X.

One "step" is one pass of the hot path over one batch of synthetic input: for
the default workload, one aligned device-to-device copy of 1 GiB of seeded
random bytes (source and destination 256-byte aligned, resident in HBM before
the clock starts).  The metric is algorithmic GB/s, read + written bytes
(copy of N bytes = 2 N, fill of N bytes = N), and its fraction of the 8 TB/s
HBM3E peak.  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

Workloads: copy (default, the headline), fill, misaligned, batch, rect, and calib (a
plain torch copy_ of the same size: not this library, only the known-size
kernel that scales the profiler's HBM counters).  Whatever the
workload, the line also carries the other configurations' figures under
"also" (measured outside the timed region), the roofline of the dominant
kernel, and the CPU baseline (the reference's host path: memcpy / dword fill,
timed on this box's cores on a bounded sample).
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
GIB = 1 << 30
MIB = 1 << 20
FILL_VALUE = 0xA5C30F1E


# Launches that bring the device out of idle before anything is timed (see --warmup).
WARMUP_AFTER_IDLE = 60


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    # After an idle period the first ~50 launches of a streaming kernel run up to 25 % slow (a hump
    # that peaks around the tenth launch and is gone by the fiftieth, whatever the kernel): the
    # default warm-up covers it.
    ap.add_argument("--warmup", type=int, default=WARMUP_AFTER_IDLE)
    ap.add_argument("--workload", default="copy",
                    choices=["copy", "fill", "misaligned", "batch", "rect", "calib", "idle_series", "batch_layouts",
                             "sustain", "pieces", "rect_grid", "rect_check", "misaligned_classes"])
    ap.add_argument("--bytes", type=int, default=GIB, help="transfer size of the copy/fill workloads")
    ap.add_argument("--rect", default="8192,131072,262144,0,0",
                    help="shape of the rect workload: rows,width,pitch[,source x,destination x] in bytes")
    ap.add_argument("--path", default="aql", choices=["aql", "hip"],
                    help="submission path of the idle_series workload")
    ap.add_argument("--tune", default="",
                    help="overrides of the launch heuristics for the timed workload, as field=value pairs of "
                         "mi355_blit_tuning_t separated by commas (e.g. store_policy=2,xcd_run=1)")
    ap.add_argument("--constant-bytes", action="store_true",
                    help="idle_series: copy a source of constant bytes instead of the workload's seeded random ones")
    ap.add_argument("--settle-ms", type=float, default=60.0,
                    help="milliseconds of back-to-back launches of the workload in front of the warm-up, which bring "
                         "the device from idle to its sustained clocks (reported in the line; 0 = none)")
    ap.add_argument("--no-sample", action="store_true", help="do not sample the clocks from sysfs around the timed region")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-verify", action="store_true",
                    help="skip the check of the timed workload's result (for runs under a profiler, whose trace "
                         "would otherwise record the check's own kernels: 200,000 of them for the batch)")
    ap.add_argument("--no-also", action="store_true", help="skip the secondary configurations")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="CPU baseline budget")
    return ap.parse_args()


def aligned_ptr(t, a=256):
    p = t.data_ptr()
    return p + (-p) % a


def seeded_bytes(n, seed):
    import numpy as np
    return np.random.default_rng(seed).integers(0, 256, n, dtype=np.uint8)


def device_bytes(torch, n, seed=None):
    """n + 512 bytes of device memory; with a seed, n seeded uniform random
    bytes from the first 256-byte boundary on, drawn on the device (a seeded
    generator of the device's own: the host stays out of it, and the GPU is not
    left idle for the seconds a host-side draw and upload of a GiB take)."""
    t = torch.empty(n + 512, dtype=torch.uint8, device="cuda:0")
    if seed is not None:
        g = torch.Generator(device="cuda:0")
        g.manual_seed(seed)
        off = (-t.data_ptr()) % 256
        t[off:off + n].random_(0, 256, generator=g)
    torch.cuda.synchronize()
    return t


SAMPLER_SOURCE = r"""
import glob, os, sys, time, json, signal
period = float(sys.argv[1])
paths = {}
for card in sorted(glob.glob('/sys/class/drm/card*/device')):
    if os.path.exists(card + '/pp_dpm_sclk'):
        paths = {'sclk': card + '/pp_dpm_sclk', 'mclk': card + '/pp_dpm_mclk'}
        power = glob.glob(card + '/hwmon/hwmon*/power1_input') + glob.glob(card + '/hwmon/hwmon*/power1_average')
        if power:
            paths['power_uW'] = power[0]
        break
cols = sorted(paths)
def current(path):
    try:
        text = open(path).read()
    except OSError:
        return None
    for line in text.splitlines():
        if line.strip().endswith('*'):
            return line.split(':')[1].strip().rstrip('*').strip()
    return text.strip()[:32]
stop = []
signal.signal(signal.SIGTERM, lambda *a: stop.append(1))
samples = []
while not stop and len(samples) < 400000:
    samples.append([time.perf_counter()] + [current(paths[k]) for k in cols])
    time.sleep(period)
json.dump({'columns': cols, 'samples': samples}, sys.stdout)
"""


class SysfsSampler:
    """The clocks and the power the driver reports for the first GPU, read from
    sysfs every `period` seconds while a measurement runs -- by a process of
    its own, which never touches the GPU: a sampling thread in this process
    would take the interpreter lock from the thread that launches and waits
    (measured: 1.5 us per step of a 20-step timed region).  Its clock,
    time.perf_counter, is the system's monotonic clock and so the same as this
    process's."""

    def __init__(self, period=0.002):
        self.period = period
        self.proc = None
        self.cols, self.samples = [], []

    def columns(self):
        return self.cols

    def start(self):
        import subprocess
        # the sampler is no part of what a profiler wrapped around this process should see
        env = {k: v for k, v in os.environ.items()
               if k != "LD_PRELOAD" and not k.startswith(("ROCP", "ROCPROF", "HSA_TOOLS"))}
        self.proc = subprocess.Popen([sys.executable, "-c", SAMPLER_SOURCE, str(self.period)], stdout=subprocess.PIPE,
                                     stderr=subprocess.DEVNULL, text=True, env=env)
        return self

    def stop(self):
        if self.proc:
            self.proc.terminate()
            try:
                out, _ = self.proc.communicate(timeout=20)
                got = json.loads(out)
                self.cols, self.samples = got["columns"], [tuple(x) for x in got["samples"]]
            except Exception:  # a sampler that fails costs the line its clock columns, nothing else
                self.proc.kill()
            self.proc = None
        return self

    def changes(self, t0, t1=None):
        """The samples between t0 and t1 that differ from the one before, as
        [ms since t0, columns...]."""
        out, last = [], None
        for smp in self.samples:
            if smp[0] < t0 - 0.003 or (t1 is not None and smp[0] > t1 + 0.003):
                continue
            if smp[1:] != last:
                out.append([round((smp[0] - t0) * 1e3, 1)] + list(smp[1:]))
                last = smp[1:]
        return out


class Runner:
    def __init__(self, torch, pkg):
        self.torch = torch
        self.capi = pkg.capi
        self.blit = pkg.capi.Blit(0)
        # a stream torch can time: events are recorded on the stream the
        # kernels are launched on
        self.tstream = torch.cuda.Stream()
        self.stream = self.tstream.cuda_stream
        assert self.stream, "need a non-null stream"

    def device_bytes(self, n, seed=None):
        return device_bytes(self.torch, n, seed)

    def time_launches(self, fn, steps, warmup):
        """W untimed + K timed back-to-back launches.  Returns (wall seconds for
        the K steps, average device microseconds per launch from HIP events on
        the launch stream)."""
        torch = self.torch
        for _ in range(warmup):
            fn()
        self.tstream.synchronize()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record(self.tstream)
        for _ in range(steps):
            fn()
        e1.record(self.tstream)
        t_issued = time.perf_counter()
        # the host watches for the closing event instead of sleeping on it: a blocked wait's wake-up is a few
        # tens of microseconds of a 6 ms region; the synchronisation behind it then returns at once
        while not e1.query():
            pass
        t_seen = time.perf_counter()
        # one device-wide synchronisation closes the region (it covers the launch stream; a stream synchronisation
        # in front of it cost another 15-20 us of host time on a device that is already idle)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        device_us = e0.elapsed_time(e1) * 1e3
        # where the wall clock's microseconds beyond the device's own lie
        self.last_wall_breakdown_us = {
            "all_steps_issued_after": round((t_issued - t0) * 1e6, 1),
            "closing_event_seen_after": round((t_seen - t0) * 1e6, 1),
            "synchronisation_returned_after": round((t1 - t0) * 1e6, 1),
            "device_first_to_last_event": round(device_us, 1)}
        return t1 - t0, device_us / steps

    def settle(self, fn, min_ms):
        """Back-to-back launches of the workload until min_ms of them have run:
        brings the device from idle to its sustained state (clocks, power) before
        anything is timed.  Returns (launches, milliseconds)."""
        t0 = time.perf_counter()
        n = 0
        while (time.perf_counter() - t0) * 1e3 < min_ms:
            for _ in range(8):
                fn()
            n += 8
            self.tstream.synchronize()
        return n, (time.perf_counter() - t0) * 1e3

    def time_settled(self, fn, steps, settle_ms=40.0, warmup=5):
        """time_launches behind a settle burst: what the secondary figures use."""
        self.settle(fn, settle_ms)
        return self.time_launches(fn, steps, warmup)

    def time_each(self, fn, steps, warmup):
        """Durations of `steps` consecutive launches, one by one: an event is
        recorded between every two launches, so each figure includes the few
        microseconds an event costs the queue (the averaged figure of
        time_launches does not).  Returns microseconds."""
        torch = self.torch
        for _ in range(warmup):
            fn()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
        ev[0].record(self.tstream)
        for i in range(steps):
            fn()
            ev[i + 1].record(self.tstream)
        self.tstream.synchronize()
        return [ev[i].elapsed_time(ev[i + 1]) * 1e3 for i in range(steps)]

    def check(self, st, what):
        self.capi.check(st, what)


def make_copy(r, nbytes, s_off=0, d_off=0):
    src = r.device_bytes(nbytes + 64, seed=0xB1170003)
    dst = r.device_bytes(nbytes + 64)
    S, D = aligned_ptr(src) + s_off, aligned_ptr(dst) + d_off
    fn = lambda: r.check(r.blit.copy(D, S, nbytes, r.stream), "copy")

    def verify():
        # device compare of the whole range (the parity tests hold the oracle comparison)
        so = (-src.data_ptr()) % 256 + s_off
        do = (-dst.data_ptr()) % 256 + d_off
        assert r.torch.equal(dst[do:do + nbytes], src[so:so + nbytes]), "copy result differs"
    return fn, verify, 2 * nbytes, (src, dst)


def make_calib(r, nbytes):
    """torch's own elementwise copy kernel: nbytes read + nbytes written."""
    src = r.device_bytes(nbytes + 64, seed=0xB1170003)
    dst = r.device_bytes(nbytes + 64)
    a, b = src[:nbytes], dst[:nbytes]

    def fn():
        with r.torch.cuda.stream(r.tstream):
            b.copy_(a)
    return fn, (lambda: None), 2 * nbytes, (src, dst)


def make_fill(r, nbytes):
    dst = r.device_bytes(nbytes + 64)
    D = aligned_ptr(dst)
    fn = lambda: r.check(r.blit.fill32(D, FILL_VALUE, nbytes // 4, r.stream), "fill32")

    def verify():
        do = (-dst.data_ptr()) % 256
        body = dst[do:do + nbytes].view(r.torch.int32)
        want = FILL_VALUE - (1 << 32)
        assert int(body.min()) == want and int(body.max()) == want, "fill result differs"
    return fn, verify, nbytes, (dst,)


def batch_layout(n=65536, arena=8 * GIB):
    """Where the batch workload's copies lie: lengths 64 B .. 256 KiB
    log-uniform, byte offsets 0..15 drawn independently for source and
    destination, regions carved one behind the other (length rounded up to 256
    plus a 256-byte guard) with the strides scaled so that the n regions fill
    an `arena`-byte source and an `arena`-byte destination.  Returns (lens, so,
    do, offs, stride): copy i moves lens[i] bytes from arena offset offs[i] +
    so[i] of the source to offs[i] + do[i] of the destination."""
    import numpy as np
    rng = np.random.default_rng(0xB1170005)
    lens = np.floor(64 * 2.0 ** (12 * rng.random(n))).astype(np.int64)
    so = rng.integers(0, 16, n)
    do = rng.integers(0, 16, n)
    need = ((lens + 255) // 256) * 256 + 256
    scale = (arena - 4096) / float(need.sum())
    stride = (np.floor(need * scale).astype(np.int64) // 256) * 256
    offs = np.concatenate([[0], np.cumsum(stride)[:-1]]) + 256
    return lens, so, do, offs, stride


def make_batch(r, n=65536, arena=8 * GIB):
    """65,536 copies, 64 B .. 256 KiB log-uniform, byte offsets 0..15 on both
    sides, non-overlapping regions spread over an `arena`-byte source and an
    `arena`-byte destination (16 GiB in all)."""
    lens, so, do, offs, _stride = batch_layout(n, arena)
    src = r.torch.empty(arena + 512, dtype=r.torch.uint8, device="cuda:0")
    dst = r.torch.empty(arena + 512, dtype=r.torch.uint8, device="cuda:0")
    # seeded 64 MiB block repeated: cheap to make, every region still has varied bytes
    blk = seeded_bytes(64 * MIB, 0xB1170005)
    blk_d = r.torch.from_numpy(blk).to("cuda:0")
    for lo in range(0, arena, blk.size):
        src[lo:lo + blk.size].copy_(blk_d[:min(blk.size, arena - lo)])
    dst.zero_()
    r.torch.cuda.synchronize()
    S, D = aligned_ptr(src), aligned_ptr(dst)
    descs = (r.capi.Desc * n)()
    for i in range(n):
        descs[i].dst = D + int(offs[i] + do[i])
        descs[i].src = S + int(offs[i] + so[i])
        descs[i].bytes = int(lens[i])
    fn = lambda: r.check(r.blit.copy_batch(descs, n, False, r.stream), "copy_batch")

    def verify():
        """Every one of the n copies against its source, on the device (the
        comparison with the oracle's bytes, guards included, is the parity
        suite's: tests/test_gpu_parity.py lays the same batch out and checks
        all 8 GiB of the destination)."""
        sh = (-src.data_ptr()) % 256
        dh = (-dst.data_ptr()) % 256
        bad = r.torch.zeros(1, dtype=r.torch.int64, device="cuda:0")
        for i in range(n):
            a = dst[dh + int(offs[i] + do[i]):dh + int(offs[i] + do[i] + lens[i])]
            b = src[sh + int(offs[i] + so[i]):sh + int(offs[i] + so[i] + lens[i])]
            bad += (a != b).any()
        assert int(bad.item()) == 0, "%d of the %d batched copies differ from their source" % (int(bad.item()), n)
        # nothing was written between the regions: the bytes that are not zero are at most the copies' own
        assert int((dst != 0).sum().item()) <= int(lens.sum()), "bytes written outside the copies"
    return fn, verify, int(2 * lens.sum()), (src, dst, descs)


def batch_layouts(r, n=65536, arena=8 * GIB):
    """Where a batch's time goes, from the product path alone: the benchmark's
    65,536 copies laid out in other ways, and other batches of the same size,
    each timed like the headline (20 back-to-back submissions behind the
    warm-up) and checked on a sample of 512 copies.  The arenas are the
    benchmark's: 8 GiB of source, 8 GiB of destination."""
    import numpy as np
    lens, so, do, offs, _stride = batch_layout(n, arena)
    src = r.torch.empty(arena + 512, dtype=r.torch.uint8, device="cuda:0")
    dst = r.torch.empty(arena + 512, dtype=r.torch.uint8, device="cuda:0")
    blk_d = r.torch.from_numpy(seeded_bytes(64 * MIB, 0xB1170005)).to("cuda:0")
    for lo in range(0, arena, 64 * MIB):
        src[lo:lo + 64 * MIB].copy_(blk_d[:min(64 * MIB, arena - lo)])
    r.torch.cuda.synchronize()
    S, D = aligned_ptr(src), aligned_ptr(dst)
    sh, dh = S - src.data_ptr(), D - dst.data_ptr()
    need = ((lens + 255) // 256) * 256 + 256
    packed = np.concatenate([[0], np.cumsum(need)[:-1]]) + 256

    def clustered(cluster_bytes):
        """Dense clusters of about cluster_bytes, the clusters spread evenly over the arena."""
        out = np.empty(n, dtype=np.int64)
        gap_ratio = (arena - 4096) / float(need.sum())
        at, start, filled = 256, 0, 0
        for i in range(n):
            if filled >= cluster_bytes:
                start = start + int(filled * gap_ratio) // 4096 * 4096
                at, filled = start + 256, 0
            out[i] = at
            at += int(need[i])
            filled += int(need[i])
        assert at < arena
        return out

    zero = so * 0
    whole = (lens // 4096 + 1) * 4096
    even = np.full(n, 32 * 1024, dtype=np.int64)
    layouts = [
        ("benchmark: spread over the arenas, byte offsets 0..15", offs, so, do, lens),
        ("the same copies packed, 256-byte gaps", packed, so, do, lens),
        ("the same copies in dense clusters of 2 MiB spread over the arenas", clustered(2 * MIB), so, do, lens),
        ("the same copies in dense clusters of 512 KiB spread over the arenas", clustered(512 * 1024), so, do, lens),
        ("benchmark placement, source and destination 256-byte aligned", offs, zero, zero, lens),
        ("benchmark placement, aligned, lengths rounded up to whole 4 KiB chunks", offs, zero, zero, whole),
        ("65,536 copies of 32 KiB, contiguous", np.arange(n, dtype=np.int64) * 32768, zero, zero, even),
        ("8,192 copies of 256 KiB, contiguous", np.arange(8192, dtype=np.int64) * 262144, zero[:8192], zero[:8192],
         np.full(8192, 262144, dtype=np.int64)),
        ("1 copy of 2 GiB", np.zeros(1, dtype=np.int64), zero[:1], zero[:1], np.full(1, 2 * GIB, dtype=np.int64)),
    ]
    rng = np.random.default_rng(0xB1170105)
    out = {}
    for name, at, s_off, d_off, ln in layouts:
        m = len(ln)
        descs = (r.capi.Desc * m)()
        for i in range(m):
            descs[i].dst = D + int(at[i] + d_off[i])
            descs[i].src = S + int(at[i] + s_off[i])
            descs[i].bytes = int(ln[i])
        fn = lambda: r.check(r.blit.copy_batch(descs, m, False, r.stream), "copy_batch")
        dst.zero_()
        r.torch.cuda.synchronize()
        _, us = r.time_settled(fn, 20)
        for i in (range(m) if m <= 512 else rng.integers(0, m, 512)):
            a = dst[dh + int(at[i] + d_off[i]):dh + int(at[i] + d_off[i] + ln[i])]
            b = src[sh + int(at[i] + s_off[i]):sh + int(at[i] + s_off[i] + ln[i])]
            assert r.torch.equal(a, b), "%s: copy %d differs" % (name, i)
        algo = 2 * int(ln.sum())
        out[name] = {"us_per_batch": round(us, 1), "bytes": algo, "gbs": round(algo / us / 1e3, 1),
                     "frac_of_peak": round(algo / us / 1e3 / HBM_PEAK_GBS, 4)}
    fn = lambda: r.check(r.blit.copy(D, S, 2 * GIB, r.stream), "copy")
    _, us = r.time_settled(fn, 20)
    out["for comparison: linear copy of 2 GiB"] = {"us_per_launch": round(us, 1), "bytes": 4 * GIB,
                                                  "gbs": round(4 * GIB / us / 1e3, 1),
                                                  "frac_of_peak": round(4 * GIB / us / 1e3 / HBM_PEAK_GBS, 4)}
    return out


def make_batch_device(r):
    """The same 65,536 copies with the descriptors resident in device memory
    (as a kernel would have left them) and no bound on their sizes given."""
    import numpy as np
    fn, verify, algo, (src, dst, descs) = make_batch(r)
    n = len(descs)
    dev = r.torch.from_numpy(np.frombuffer(bytes(descs), dtype=np.uint8).copy()).to("cuda:0")
    r.torch.cuda.synchronize()
    fn_dev = lambda: r.check(r.blit.copy_batch(dev.data_ptr(), n, True, r.stream), "copy_batch, device descriptors")
    return fn_dev, verify, algo, (src, dst, descs, dev)


def make_rect(r, rows=8192, width=128 * 1024, pitch=256 * 1024, s_x=0, d_x=0):
    """rows x width bytes out of two pitched 2-D surfaces (rows x pitch each),
    the region starting s_x / d_x bytes into each row."""
    import numpy as np
    total = rows * pitch
    src = r.torch.empty(total + 512, dtype=r.torch.uint8, device="cuda:0")
    dst = r.torch.empty(total + 512, dtype=r.torch.uint8, device="cuda:0")
    blk = seeded_bytes(min(64 * MIB, total), 0xB1170006)
    blk_d = r.torch.from_numpy(blk).to("cuda:0")
    for lo in range(0, total, blk.size):
        m = min(blk.size, total - lo)
        src[lo:lo + m].copy_(blk_d[:m])
    dst.zero_()
    r.torch.cuda.synchronize()
    S, D = aligned_ptr(src), aligned_ptr(dst)
    sp, dp = (S, pitch, 0), (D, pitch, 0)
    fn = lambda: r.check(r.blit.copy_rect(dp, (d_x, 0, 0), sp, (s_x, 0, 0), (width, rows, 1), r.stream), "copy_rect")

    def verify():
        sh = (-src.data_ptr()) % 256
        dh = (-dst.data_ptr()) % 256
        s2 = src[sh:sh + total].view(rows, pitch)
        d2 = dst[dh:dh + total].view(rows, pitch)
        assert r.torch.equal(d2[:, d_x:d_x + width], s2[:, s_x:s_x + width]), "rect copy differs"
        assert int(d2[:, :d_x].max().item() if d_x else 0) == 0, "rect copy wrote in front of the region"
        if d_x + width < pitch:
            assert int(d2[:, d_x + width:].max().item()) == 0, "rect copy wrote behind the region"
    return fn, verify, 2 * rows * width, (src, dst)


RECT_SHAPES = (
    # rows, width, pitch, src x, dst x: 1 GiB moved each (the last two 256 MiB); the third has a pitch that is
    # not a power of two
    (8192, 128 * 1024, 256 * 1024, 0, 0),
    (8192, 128 * 1024 - 7, 256 * 1024 + 4, 3, 9),
    (8192, 128 * 1024, 260 * 1024, 0, 0),
    (262144, 4096, 8192, 0, 0),
    (1048576, 1024, 2048, 0, 0),
    (1048576, 256, 512, 0, 0),
    (1048576, 64, 256, 0, 0),
)


def rect_shapes(r):
    out = {}
    for rows, width, pitch, sx, dx in RECT_SHAPES:
        fn, verify, algo, keep = make_rect(r, rows, width, pitch, sx, dx)
        _, us = r.time_settled(fn, 20)
        verify()
        rec = {"gbs": round(algo / us / 1e3, 1), "us_per_launch": round(us, 2),
               "unroll": r.blit.last_plan().unroll}
        # HBM bytes per launch from the committed counter runs, where this shape has one: rows that
        # use part of every 128-byte line they touch move more bytes than they copy
        traffic = load_traffic("rect_%dx%d_%d" % (rows, width, pitch)) if (sx, dx) == (0, 0) else None
        if traffic:
            rec["hbm_traffic_gbs"] = round(traffic / us / 1e3, 1)
        out["%dx%d/%d+%d,%d" % (rows, width, pitch, sx, dx)] = rec
        del fn, verify, keep
        r.torch.cuda.empty_cache()
    return out


def size_sweep(r):
    """Aligned copy and fill at 4 KiB -> 4 GiB in powers of 4: microseconds per
    launch (HIP events around back-to-back launches) and algorithmic GB/s.
    Sizes up to a few hundred MiB are helped by the 256 MiB last-level cache."""
    out = {"copy": {}, "fill": {}}
    top = 4 * GIB
    src = r.device_bytes(top + 64, seed=None)
    dst = r.device_bytes(top + 64)
    src.random_(0, 256)
    r.torch.cuda.synchronize()
    S, D = aligned_ptr(src), aligned_ptr(dst)
    for k in range(11):
        n = 4096 * 4 ** k
        iters = 100 if n <= MIB else (30 if n <= 256 * MIB else 8)
        _, us = r.time_settled(lambda: r.check(r.blit.copy(D, S, n, r.stream), "copy"), iters)
        out["copy"][str(n)] = {"us": round(us, 2), "gbs": round(2 * n / us / 1e3, 1)}
        _, us = r.time_settled(lambda: r.check(r.blit.fill32(D, FILL_VALUE, n // 4, r.stream), "fill32"), iters)
        out["fill"][str(n)] = {"us": round(us, 2), "gbs": round(n / us / 1e3, 1)}
    so, do = (-src.data_ptr()) % 256, (-dst.data_ptr()) % 256
    r.check(r.blit.copy(D, S, top, r.stream), "copy")
    r.tstream.synchronize()
    assert r.torch.equal(dst[do:do + top], src[so:so + top]), "4 GiB copy differs"
    return out


def misaligned_figures(r, pkg):
    """BASELINE's misaligned configuration in full: a 1 GiB - 64 B copy for one
    offset pair of every class the kernels distinguish -- (src - dst) & 3 picks
    the kernel (0: dword-aligned loads, else realignment), (src - dst) & 12
    where the source sits in its 16 bytes -- plus the headline pair (3, 9); a
    length sweep 1 B .. 64 MiB at (3, 9), back-to-back launches; and the
    blocking 4 KiB copy at (3, 9) on both submission paths.  Every copy is
    compared with its source."""
    torch = r.torch
    n = GIB - 64
    src = r.device_bytes(GIB + 64, seed=0xB1170004)
    dst = r.device_bytes(GIB + 64)
    S, D = aligned_ptr(src), aligned_ptr(dst)
    sh, dh = S - src.data_ptr(), D - dst.data_ptr()

    def same(so, do, m):
        return torch.equal(dst[dh + do:dh + do + m], src[sh + so:sh + so + m])

    out = {"classes_1GiB": {}, "length_sweep_3_9": {}, "blocking_4KiB_us": {}}
    pairs = [((9 + c) & 15, 9) for c in range(8)] + [(3, 9)]
    for so, do in pairs:
        fn = lambda: r.check(r.blit.copy(D + do, S + so, n, r.stream), "copy")
        _, us = r.time_settled(fn, 20)
        assert same(so, do, n), "misaligned copy (%d, %d) differs" % (so, do)
        out["classes_1GiB"]["src&15=%d,dst&15=%d" % (so, do)] = {
            "shift": (so - do) & 3, "src_slot": (so - do) & 12, "us_per_launch": round(us, 2),
            "gbs": round(2 * n / us / 1e3, 1), "frac_of_peak": round(2 * n / us / 1e3 / HBM_PEAK_GBS, 4)}
    for m in (1, 64, 1024, 16 * 1024, 256 * 1024, 4 * MIB, 64 * MIB):
        dst[dh:dh + m + 64].zero_()
        fn = lambda: r.check(r.blit.copy(D + 9, S + 3, m, r.stream), "copy")
        _, us = r.time_settled(fn, 100 if m <= 4 * MIB else 30)
        assert same(3, 9, m) and int(dst[dh + 9 + m]) == 0 and int(dst[dh + 8]) == 0, "misaligned copy of %d bytes differs" % m
        out["length_sweep_3_9"][str(m)] = {"us_per_launch": round(us, 2), "gbs": round(2 * m / us / 1e3, 2)}
    ts = []
    for i in range(220):
        t0 = time.perf_counter()
        r.check(r.blit.copy(D + 9, S + 3, 4096), "copy")
        r.check(r.blit.synchronize(), "synchronize")
        ts.append(time.perf_counter() - t0)
    ts = sorted(ts[20:])
    out["blocking_4KiB_us"]["hip"] = round(ts[len(ts) // 2] * 1e6, 2)
    eng = pkg.aql.AqlBlit(0)
    sig = pkg.aql.HsaSignals()
    try:
        c = sig.create(1)
        ts = []
        for i in range(220):
            sig.store(c, 1)
            t0 = time.perf_counter()
            r.check(eng.copy(D + 9, S + 3, 4096, completion=c), "copy")
            sig.wait_below_one(c)
            ts.append(time.perf_counter() - t0)
        ts = sorted(ts[20:])
        out["blocking_4KiB_us"]["aql"] = round(ts[len(ts) // 2] * 1e6, 2)
        sig.destroy(c)
    finally:
        eng.close()
    assert same(3, 9, 4096)
    out["how"] = ("1 GiB - 64 B per class: HIP events around 20 back-to-back launches behind a settle burst; length sweep: "
                  "the same with 100 launches (30 at 64 MiB), launch-bound below a few MiB; blocking: submit to completion "
                  "seen by the host, median of 200, through the Python binding")
    return out


def sustain_series(r):
    """Whether a long transfer is slower per byte than a short one, and why: in
    one process, back-to-back aligned copies of 1 GiB (272 commands), of 4 GiB
    as a single launch (68 commands: the same bytes, the same ~86 ms of load),
    of 4 GiB the way the library submits it (eight launches of 512 MiB a
    command) and of 1 GiB again, each series after a second without work, every
    command timed by an event behind it, with the clocks the driver reports
    sampled every millisecond.  Under `rocprofv3 --kernel-trace` the trace holds
    the kernels' own durations for the same launches."""
    torch = r.torch
    top = 4 * GIB
    src = r.device_bytes(top + 64, seed=0xB1170003)
    dst = r.device_bytes(top + 64)
    S, D = aligned_ptr(src), aligned_ptr(dst)
    out = {"metric": "pace of back-to-back aligned copies, 1 GiB against 4 GiB", "unit": "us per GiB", "series": []}
    sampler = SysfsSampler(0.001).start()
    windows = []
    for gib, launches, one_launch in ((1, 272, False), (4, 68, True), (4, 68, False), (1, 272, False)):
        n = gib * GIB
        fn = lambda: r.check(r.blit.copy(D, S, n, r.stream), "copy")
        r.blit.set_tuning(copy_piece_mib=1) if one_launch else r.blit.set_tuning()
        r.tstream.synchronize()
        torch.cuda.synchronize()
        time.sleep(1.0)
        t0 = time.perf_counter()
        us = r.time_each(fn, launches, 0)
        windows.append((t0, time.perf_counter()))
        per_gib = [u / gib for u in us]
        k = launches // 4

        def mean(v):
            return round(sum(v) / len(v), 2)
        out["series"].append({
            "copy_GiB": gib, "commands": launches, "launches_per_command": r.blit.last_plan().pieces,
            "us_per_GiB_by_quarter_of_the_series": [mean(per_gib[i * k:(i + 1) * k]) for i in range(4)],
            "us_per_GiB_last_half": mean(per_gib[launches // 2:]),
            "us_per_GiB_min": round(min(per_gib), 2),
            "us_per_launch": [round(u, 1) for u in us]})
    r.blit.set_tuning()
    sampler.stop()
    for series, (t0, t1) in zip(out["series"], windows):
        series["sysfs_columns"] = ["ms since first launch"] + sampler.columns()
        series["sysfs_changes"] = sampler.changes(t0, t1)
    so, do = (-src.data_ptr()) % 256, (-dst.data_ptr()) % 256
    assert torch.equal(dst[do:do + top], src[so:so + top]), "4 GiB copy differs"
    return out


def piece_sweep(r, rounds=3):
    """What cutting a long copy into consecutive launches is worth: copies of 1 to
    8 GiB, aligned and at byte offsets (3, 9), each as one launch and in pieces
    of 2 GiB down to 128 MiB (the tuning field copy_piece_mib), through the
    library's own entry point.  Every configuration is timed `rounds` times in
    rotation, 24 GiB of copies a time behind a settle burst; the figure is the
    median, in microseconds per GiB, from events on the launch stream."""
    torch = r.torch
    top = 8 * GIB
    src = r.device_bytes(top + 64, seed=0xB1170003)
    dst = r.device_bytes(top + 64)
    S, D = aligned_ptr(src), aligned_ptr(dst)
    cases = []
    for gib in (1, 2, 4, 8):
        for s_off, d_off in ((0, 0), (3, 9)):
            if (s_off, d_off) != (0, 0) and gib not in (1, 4):
                continue
            for piece_mib in (1, 2048, 1024, 512, 256, 128):
                if piece_mib != 1 and piece_mib >= gib * 1024:
                    continue
                cases.append({"copy_GiB": gib, "offsets": [s_off, d_off], "copy_piece_mib": piece_mib, "us_per_GiB": []})
    for _ in range(rounds):
        for c in cases:
            n = c["copy_GiB"] * GIB - 64
            s_off, d_off = c["offsets"]
            fn = lambda: r.check(r.blit.copy(D + d_off, S + s_off, n, r.stream), "copy")
            r.blit.set_tuning(copy_piece_mib=c["copy_piece_mib"])
            _, us = r.time_settled(fn, max(3, 24 // c["copy_GiB"]), settle_ms=30.0, warmup=2)
            c["launches"] = r.blit.last_plan().pieces
            c["us_per_GiB"].append(round(us * GIB / n, 2))
    r.blit.set_tuning()
    for c in cases:
        c["median"] = sorted(c["us_per_GiB"])[len(c["us_per_GiB"]) // 2]
    # what the library does by itself
    default = []
    for gib in (1, 2, 4, 8):
        n = gib * GIB - 64
        fn = lambda: r.check(r.blit.copy(D, S, n, r.stream), "copy")
        _, us = r.time_settled(fn, max(3, 24 // gib), settle_ms=30.0, warmup=2)
        default.append({"copy_GiB": gib, "launches": r.blit.last_plan().pieces, "us_per_GiB": round(us * GIB / n, 2)})
    # where a single long launch loses: single launches of 1 and 4 GiB timed one by one, back to back and with the
    # stream drained and the host asleep between them; and the 4 GiB launch in launch order and with other run lengths
    def one_by_one(n, launches, gap_s, **tuning):
        r.blit.set_tuning(copy_piece_mib=1, **tuning)
        fn = lambda: r.check(r.blit.copy(D, S, n, r.stream), "copy")
        r.settle(fn, 30.0)
        ev = []
        for _ in range(launches):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(r.tstream)
            fn()
            e1.record(r.tstream)
            ev.append((e0, e1))
            if gap_s is not None:
                r.tstream.synchronize()
                time.sleep(gap_s)
        r.tstream.synchronize()
        us = sorted(a.elapsed_time(b) * 1e3 * GIB / n for a, b in ev)
        return {"median": round(us[len(us) // 2], 2), "min": round(us[0], 2), "max": round(us[-1], 2)}
    single = []
    for gib in (1, 4):
        for gap_ms in (None, 0.5, 5.0):
            single.append({"copy_GiB": gib, "idle_ms_between_launches": gap_ms,
                           "us_per_GiB": one_by_one(gib * GIB, 48 // gib, None if gap_ms is None else gap_ms * 1e-3)})
    orders = [{"copy_GiB": 4, "xcd_run": x, "us_per_GiB": one_by_one(4 * GIB, 12, None, xcd_run=x)}
              for x in (1, 288, 576, 1152, 4608)]
    r.blit.set_tuning()
    so, do = (-src.data_ptr()) % 256, (-dst.data_ptr()) % 256
    assert torch.equal(dst[do:do + top - 64], src[so:so + top - 64]), "8 GiB copy differs"
    return {"cases": cases, "default": default, "single_launches": single, "single_launch_walk_orders": orders}


RECT_GRID_WIDTHS_KIB = (2, 4, 8, 12, 16, 24, 32, 48, 64, 96, 128, 256)
RECT_GRID_RATIOS = (2, 3, 4, 6, 8, 12, 16)
# shapes off that grid, to check rules read from it: widths that are not on it at pitches 2.5 to 10 times the
# width, odd widths at power-of-two pitches, pitches a line off a power of two, and a few of the grid's own
RECT_CHECK_SHAPES_KIB = tuple((w, w * r) for w in (3, 5, 6, 10, 20, 40, 80, 160) for r in (2.5, 3.5, 5, 7, 10)) + (
    (6, 16), (6, 32), (10, 32), (10, 64), (20, 64), (20, 128), (40, 128), (40, 256), (80, 256), (80, 512), (160, 512),
    (20, 256), (40, 512), (16, 64.25), (32, 128.25), (64, 256.25), (128, 512.25), (8, 16.25), (32, 512.25), (16, 48.25),
    (48, 192), (32, 192), (96, 384), (8, 16), (32, 512), (16, 256))


def rect_grid(r, which):
    """Where the region copy's heuristics stand: rows of whole cache lines,
    512 MiB moved per launch (less where 12 GiB of surface do not hold it), each
    shape as the library plans it and at eight forced combinations of store
    policy (nt, sc1) and walk order (launch order, XCD runs of 144, 576 and 2304
    units).  One JSON object per shape, GB/s of bytes read plus written."""
    K = 1024
    if which == "check":
        pairs = [(int(w * K) // 128 * 128, int(p * K) // 128 * 128) for w, p in RECT_CHECK_SHAPES_KIB]
    else:
        pairs = [(w * K, w * K * ratio) for ratio in RECT_GRID_RATIOS for w in RECT_GRID_WIDTHS_KIB]
    out = []
    for width, pitch in pairs:
        rows = min(512 * MIB // width, 12 * GIB // pitch)
        fn, verify, algo, keep = make_rect(r, rows, width, pitch, 0, 0)
        r.blit.set_tuning()
        _, us = r.time_settled(fn, 12, settle_ms=15)
        plan = r.blit.last_plan()
        rec = {"width": width, "pitch": pitch, "rows": rows,
               "planned": {"store_policy": plan.store_policy, "xcd_run": plan.xcd_run, "gbs": round(algo / us / 1e3)},
               "forced_gbs": {}}
        for store, name in ((2, "nt"), (3, "sc1")):
            for run in (1, 144, 576, 2304):
                r.blit.set_tuning(xcd_run=run, store_policy=store)
                _, us = r.time_settled(fn, 12, settle_ms=5)
                rec["forced_gbs"]["%s_run%d" % (name, run)] = round(algo / us / 1e3)
        r.blit.set_tuning()
        fn()
        r.tstream.synchronize()
        verify()
        out.append(rec)
        del fn, verify, keep
        r.torch.cuda.empty_cache()
    return out


def small_copy_latency(r, sizes=(4096, 65536, MIB)):
    """Host-observed microseconds per blocking copy (submit -> completion seen),
    the way rocrtst times hsa_amd_memory_async_copy (memory_async_copy.cc:396-405)."""
    out = {}
    src = r.device_bytes(max(sizes) + 64, seed=0xB1170003)
    dst = r.device_bytes(max(sizes) + 64)
    S, D = aligned_ptr(src), aligned_ptr(dst)
    for n in sizes:
        for _ in range(20):
            r.check(r.blit.copy(D, S, n), "copy")
            r.check(r.blit.synchronize(), "synchronize")
        ts = []
        for _ in range(200):
            t0 = time.perf_counter()
            r.check(r.blit.copy(D, S, n), "copy")
            r.check(r.blit.synchronize(), "synchronize")
            ts.append(time.perf_counter() - t0)
        ts.sort()
        out[str(n)] = round(ts[len(ts) // 2] * 1e6, 2)
    return out


def aql_path(r, pkg):
    """The same workloads submitted as hand-built AQL packets on an HSA queue
    (include/mi355_blit_aql.h).  Device time per command from the packet
    processor's own timestamps in the completion signal; small copies as
    host-observed microseconds, submit -> completion signal seen."""
    import numpy as np
    aql = pkg.aql
    eng = aql.AqlBlit(0)
    sig = aql.HsaSignals()
    out = {}
    try:
        eng.enable_profiling(True)
        src = r.device_bytes(GIB + 64, seed=0xB1170003)
        dst = r.device_bytes(GIB + 64)
        S, D = aligned_ptr(src), aligned_ptr(dst)
        cases = (("copy_1GiB", lambda c: eng.copy(D, S, GIB, completion=c), 2 * GIB),
                 ("fill_1GiB", lambda c: eng.fill32(D, FILL_VALUE, GIB // 4, completion=c), GIB),
                 ("misaligned_1GiB", lambda c: eng.copy(D + 9, S + 3, GIB - 64, completion=c), 2 * (GIB - 64)))
        for key, submit, algo in cases:
            # one command at a time: with the barrier bit clear, commands
            # queued together would overlap and stretch each other's time
            sigs = [sig.create(1) for _ in range(WARMUP_AFTER_IDLE + 20)]
            for c in sigs:
                r.check(submit(c), key)
                sig.wait_below_one(c)
            us = [eng.command_time_us(c) for c in sigs[WARMUP_AFTER_IDLE:]]
            for c in sigs:
                sig.destroy(c)
            avg = sum(us) / len(us)
            out[key] = {"gbs": round(algo / avg / 1e3, 1), "frac_of_peak": round(algo / avg / 1e3 / HBM_PEAK_GBS, 4),
                        "us_per_launch": round(avg, 2)}
        so = (-src.data_ptr()) % 256 + 3
        do = (-dst.data_ptr()) % 256 + 9
        assert r.torch.equal(dst[do:do + GIB - 64], src[so:so + GIB - 64]), "AQL copy result differs"
        eng.enable_profiling(False)
        c = sig.create(1)
        for key, system_scope in (("small_copy_us", True), ("small_copy_us_agent_scope", False)):
            # system scope: the reference's fences (amd_blit_kernel.cpp:870-873); agent scope: for
            # callers whose consumers are kernels on this GPU
            eng.set_system_scope_fences(system_scope)
            lat = {}
            for n in (4096, 65536, MIB):
                ts = []
                for i in range(220):
                    sig.store(c, 1)
                    t0 = time.perf_counter()
                    r.check(eng.copy(D, S, n, completion=c), "copy")
                    sig.wait_below_one(c)
                    ts.append(time.perf_counter() - t0)
                ts = sorted(ts[20:])
                lat[str(n)] = round(ts[len(ts) // 2] * 1e6, 2)
            out[key] = lat
        eng.set_system_scope_fences(True)
        sig.destroy(c)
        del src, dst
        r.torch.cuda.empty_cache()
        # the batch, whole submission by the host clock
        hip_blit = r.blit
        fn, verify, algo, keep = make_batch(r)
        descs = keep[2]
        n = len(descs)
        for _ in range(WARMUP_AFTER_IDLE // 2):
            r.check(eng.copy_batch(descs, n), "copy_batch")
        r.check(eng.synchronize(), "wait_idle")
        t0 = time.perf_counter()
        for _ in range(20):
            r.check(eng.copy_batch(descs, n), "copy_batch")
        r.check(eng.synchronize(), "wait_idle")
        us = (time.perf_counter() - t0) / 20 * 1e6
        verify()
        lat = []
        for _ in range(15):
            t0 = time.perf_counter()
            r.check(eng.copy_batch(descs, n), "copy_batch")
            r.check(eng.synchronize(), "wait_idle")
            lat.append((time.perf_counter() - t0) * 1e6)
        out["batch_65536"] = {"gbs": round(algo / us / 1e3, 1), "frac_of_peak": round(algo / us / 1e3 / HBM_PEAK_GBS, 4),
                              "us_per_launch": round(us, 2), "blocking_us_median": round(sorted(lat)[len(lat) // 2], 1)}
        out["how"] = ("AQL packets on an HSA queue; 1 GiB cases: packet-processor timestamps of 20 commands; "
                      "batch: host clock over 20 submissions; small copies: blocking copy by the host clock through the "
                      "Python binding, submit to completion signal seen, median of 200 (the native driver's figures, "
                      "cut at the packet processor's timestamps, are in profiles/small_copy_latency.md)")
        del keep, hip_blit
    finally:
        eng.close()
    return out


def host_link(r, pkg):
    """Host <-> device through the blit kernel over the host link (pinned host
    memory, the routes of include/mi355_blit.h), with the runtime's own
    hsa_memory_copy beside it, which sends such copies to its DMA engines
    (amd_gpu_agent.cpp:2370-2377).  Blocking calls, host clock, best of 5;
    GB/s of bytes moved (not read plus written: the link carries them once)."""
    eng = pkg.aql.AqlBlit(0)
    out = {}
    try:
        hsa = C.CDLL("libhsa-runtime64.so.1")
        hsa.hsa_memory_copy.restype = C.c_int
        hsa.hsa_memory_copy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
    except (OSError, AttributeError):
        hsa = None
    try:
        for n in (16 * MIB, 256 * MIB):
            host = r.torch.empty(n, dtype=r.torch.uint8, pin_memory=True)
            host.numpy()[:] = seeded_bytes(n, 0xB1170006)
            back = r.torch.zeros(n, dtype=r.torch.uint8, pin_memory=True)
            dev = r.torch.zeros(n, dtype=r.torch.uint8, device="cuda:0")
            r.torch.cuda.synchronize()
            legs = [("h2d", lambda: eng.hsa_memory_copy(dev.data_ptr(), host.data_ptr(), n)),
                    ("d2h", lambda: eng.hsa_memory_copy(back.data_ptr(), dev.data_ptr(), n))]
            if hsa is not None:
                legs += [("reference_h2d", lambda: hsa.hsa_memory_copy(dev.data_ptr(), host.data_ptr(), n)),
                         ("reference_d2h", lambda: hsa.hsa_memory_copy(back.data_ptr(), dev.data_ptr(), n))]
            for name, fn in legs:
                best = None
                for _ in range(6):
                    t0 = time.perf_counter()
                    st = fn()
                    t = time.perf_counter() - t0
                    if st != 0:
                        best = None
                        break
                    best = t if best is None else min(best, t)
                if best:
                    out["%s_%dMiB_gbs" % (name, n // MIB)] = round(n / best / 1e9, 2)
            assert r.torch.equal(back, host), "host -> device -> host differs"
            del host, back, dev
    finally:
        eng.close()
    out["how"] = "pinned host memory, blocking calls, host clock, best of 6; reference = hsa_memory_copy of the loaded runtime (DMA engines)"
    return out


def reference_gpu_path(r):
    """The reference's own blit kernels on this GPU, for orientation: the ROCr
    this process already runs on (libhsa-runtime64, the binary build of the same
    component) serves hsa_memory_copy / hsa_amd_memory_fill on same-GPU device
    pointers with AMD::BlitKernel (runtime.cpp:513, amd_gpu_agent.cpp:951, 1285).
    Blocking calls timed with the host clock, best of a few."""
    try:
        hsa = C.CDLL("libhsa-runtime64.so.1")
        hsa.hsa_init.restype = C.c_int
        hsa.hsa_memory_copy.restype = C.c_int
        hsa.hsa_memory_copy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        hsa.hsa_amd_memory_fill.restype = C.c_int
        hsa.hsa_amd_memory_fill.argtypes = [C.c_void_p, C.c_uint32, C.c_size_t]
        if hsa.hsa_init() != 0:
            return None
    except (OSError, AttributeError):
        return None
    src = r.device_bytes(GIB + 64, seed=0xB1170003)
    dst = r.device_bytes(GIB + 64)
    S, D = aligned_ptr(src), aligned_ptr(dst)

    def best(fn, reps):
        b = 1e9
        for _ in range(reps):
            t0 = time.perf_counter()
            st = fn()
            b = min(b, time.perf_counter() - t0)
            if st != 0:
                return None
        return b

    out = {}
    t = best(lambda: hsa.hsa_memory_copy(D, S, GIB), 6)
    if t:
        assert r.torch.equal(dst[(-dst.data_ptr()) % 256:][:GIB], src[(-src.data_ptr()) % 256:][:GIB])
        out["copy_1GiB_gbs"] = round(2 * GIB / t / 1e9, 1)
    t = best(lambda: hsa.hsa_memory_copy(D + 9, S + 3, GIB - 64), 3)
    if t:
        out["misaligned_1GiB_gbs"] = round(2 * (GIB - 64) / t / 1e9, 1)
    t = best(lambda: hsa.hsa_amd_memory_fill(D, FILL_VALUE, GIB // 4), 6)
    if t:
        out["fill_1GiB_gbs"] = round(GIB / t / 1e9, 1)
    t = best(lambda: hsa.hsa_memory_copy(D, S, 4096), 200)
    if t:
        out["copy_4KiB_us"] = round(t * 1e6, 2)
    t = best(lambda: hsa.hsa_memory_copy(D, S, MIB), 200)
    if t:
        out["copy_1MiB_us"] = round(t * 1e6, 2)
    rect = reference_rect(r, hsa, S, D)
    if rect:
        out["rect_4096x128KiB_gbs"] = rect
    out["how"] = ("blocking hsa_memory_copy / hsa_amd_memory_fill of the loaded libhsa-runtime64, host clock, best of n; "
                  "region copy: hsa_amd_memory_async_copy_rect (SDMA engines), submit to completion signal")
    return out or None


def reference_rect(r, hsa, S, D):
    """The reference's region copy (SDMA engines, amd_gpu_agent.cpp:1255-1283):
    4096 rows of 128 KiB out of 256 KiB-pitch surfaces inside the 1 GiB
    buffers, device to device; GB/s of bytes read plus written."""
    try:
        import __graft_entry__ as entry
        f = hsa.hsa_amd_memory_async_copy_rect
        aql = entry.load_package().aql
        sig = aql.HsaSignals()
        eng = aql.AqlBlit(0)
        gpu = eng.lib.mi355_aql_gpu_agent(eng.handle)
        eng.close()
    except (OSError, AttributeError, RuntimeError):
        return None
    capi = r.capi
    f.restype = C.c_int
    f.argtypes = [C.POINTER(capi.PitchedPtr), C.POINTER(capi.Dim3), C.POINTER(capi.PitchedPtr), C.POINTER(capi.Dim3),
                  C.POINTER(capi.Dim3), C.c_uint64, C.c_int, C.c_uint32, C.c_void_p, C.c_uint64]
    rows, width, pitch = 4096, 128 * 1024, 256 * 1024
    sp, dp = capi.PitchedPtr(S, pitch, rows * pitch), capi.PitchedPtr(D, pitch, rows * pitch)
    zero, ext = capi.Dim3(0, 0, 0), capi.Dim3(width, rows, 1)
    done = sig.create(1)
    best = None
    for _ in range(4):
        sig.store(done, 1)
        t0 = time.perf_counter()
        if f(dp, zero, sp, zero, ext, gpu, 3, 0, None, done) != 0:   # 3 = hsaDeviceToDevice
            best = None
            break
        sig.wait_below_one(done)
        t = time.perf_counter() - t0
        best = t if best is None else min(best, t)
    sig.destroy(done)
    return round(2 * rows * width / best / 1e9, 1) if best else None


def idle_series(pkg, torch, nbytes, launches, idle_s, constant_bytes=False):
    """How a burst of back-to-back copies of nbytes settles after idle_s seconds
    without work: the pace of every launch (end of command i minus end of
    command i-1, from the packet processor's timestamps in the completion
    signals, AQL path) next to the clocks and the power the driver reports in
    sysfs, sampled every millisecond by a host thread while the burst runs.
    The source holds the headline workload's seeded bytes or, as a control,
    the same byte everywhere: what the device's power management does to a
    burst depends on how much the data toggles."""
    aql = pkg.aql
    eng = aql.AqlBlit(0)
    sig = aql.HsaSignals()
    a = device_bytes(torch, nbytes, None if constant_bytes else 0xB1170003)
    if constant_bytes:
        a.fill_(3)
    b = torch.empty(nbytes + 512, dtype=torch.uint8, device="cuda:0").fill_(5)
    A, B = aligned_ptr(a), aligned_ptr(b)
    torch.cuda.synchronize()
    eng.enable_profiling(True)
    sigs = [sig.create(1) for _ in range(launches)]
    sampler = SysfsSampler(0.001).start()
    time.sleep(idle_s)
    t0 = time.perf_counter()
    for c in sigs:
        assert eng.copy(B, A, nbytes, completion=c) == 0
    sig.wait_below_one(sigs[-1])
    t1 = time.perf_counter()
    time.sleep(0.005)
    sampler.stop()
    ends = []
    first_start = None
    for c in sigs:
        x, y, f = C.c_uint64(), C.c_uint64(), C.c_uint64()
        assert eng.lib.mi355_aql_get_command_time(eng.handle, c, C.byref(x), C.byref(y), C.byref(f)) == 0
        if first_start is None:
            first_start = x.value * 1e6 / f.value
        ends.append(y.value * 1e6 / f.value)
        sig.destroy(c)
    eng.close()
    pace = [round(ends[0] - first_start, 1)] + [round(ends[i] - ends[i - 1], 1) for i in range(1, launches)]
    return {"metric": "pace of back-to-back %d MiB copies of %s bytes after %.1f s idle, AQL path" % (
                nbytes // MIB, "constant" if constant_bytes else "seeded random", idle_s),
            "unit": "us per launch", "launches": launches, "pace_us": pace,
            "sysfs_columns": ["ms since first submit"] + sampler.columns(), "sysfs_changes": sampler.changes(t0, t1)}


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(ora, budget_s):
    """The reference's host path on this box's cores: memcpy of 256 MiB (what
    hsa_memory_copy does for host pointers, core/runtime/runtime.cpp:507-510)
    and the dword fill of the same buffer, on one thread (what the reference
    really does) and on T threads: persistent workers pinned one to a CPU, each
    with a contiguous 64-byte aligned slice whose pages it touched first.
    Bounded repetitions, best of at least 5, every byte verified afterwards."""
    import numpy as np
    n = 256 * MIB
    allowed = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    # one GPU's share of a box is 16 host threads, whatever the CPU count says
    T = max(1, min(16, allowed))
    pool = ora.oracle_pool_create(T)
    assert pool, "oracle_pool_create failed"
    T = ora.oracle_pool_threads(pool)

    def aligned(nbytes):
        raw = np.empty(nbytes + 64, dtype=np.uint8)   # untouched pages
        off = (-raw.ctypes.data) % 64
        return raw, raw[off:off + nbytes]

    raw_s, src = aligned(n)
    raw_d, dst = aligned(n)
    ora.oracle_pool_first_touch(pool, src.ctypes.data, n)   # owners touch their slices first
    ora.oracle_pool_first_touch(pool, dst.ctypes.data, n)
    ora.oracle_fill_random(src.ctypes.data, 16 * MIB, 0xB1170001)
    for lo in range(16 * MIB, n, 16 * MIB):
        ora.oracle_pool_copy(pool, src.ctypes.data + lo, src.ctypes.data, 16 * MIB)

    def best_of(fn, seconds):
        best, reps, t_end = 1e9, 0, time.perf_counter() + seconds
        while reps < 5 or (time.perf_counter() < t_end and reps < 200):
            t0 = time.perf_counter()
            fn()
            best = min(best, time.perf_counter() - t0)
            reps += 1
        return best, reps

    share = budget_s / 4.0
    out = {}
    c1, r1 = best_of(lambda: ora.oracle_copy(dst.ctypes.data, src.ctypes.data, n), share)
    assert np.array_equal(dst, src), "single-thread host copy differs"
    dst[:] = 0
    ct, rt = best_of(lambda: ora.oracle_pool_copy(pool, dst.ctypes.data, src.ctypes.data, n), share)
    assert np.array_equal(dst, src), "pooled host copy differs"
    f1, q1 = best_of(lambda: ora.oracle_fill32(dst.ctypes.data, FILL_VALUE, n // 4), share)
    assert bool((dst.view("<u4") == FILL_VALUE).all()), "single-thread host fill differs"
    dst[:] = 0
    ft, qt = best_of(lambda: ora.oracle_pool_fill32(pool, dst.ctypes.data, FILL_VALUE, n // 4), share)
    assert bool((dst.view("<u4") == FILL_VALUE).all()), "pooled host fill differs"
    pinned = ora.oracle_pool_pinned(pool)
    ora.oracle_pool_destroy(pool)
    out = {
        "value": round(2 * n / ct / 1e9, 2), "unit": "GB/s", "cores": T, "kind": "port",
        "sample": "host memcpy of 256 MiB seeded bytes on %d pinned threads (oracle_pool_copy: persistent workers, "
                  "contiguous 64-byte aligned slices first touched by their owners), best of %d, all bytes "
                  "verified; read+write bytes" % (T, rt),
        "cpu_model": cpu_model(), "cpu_count": os.cpu_count(), "cpus_allowed": allowed, "threads_pinned": pinned,
        "cores_note": "T = min(16, CPUs this process may run on): 16 host threads are one GPU's share of a box",
        "copy_1thread_gbs": round(2 * n / c1 / 1e9, 2),
        "copy_Tthreads_gbs": round(2 * n / ct / 1e9, 2),
        "fill_1thread_gbs": round(n / f1 / 1e9, 2),
        "fill_Tthreads_gbs": round(n / ft / 1e9, 2),
        "reps": {"copy_1thread": r1, "copy_Tthreads": rt, "fill_1thread": q1, "fill_Tthreads": qt},
    }
    return out


def idle_series_hip(pkg, torch, nbytes, launches, idle_s, constant_bytes=False, bursts=3):
    """The HIP path's counterpart of idle_series: `bursts` bursts of back-to-back
    copies of nbytes, each after idle_s seconds without work, every launch
    timed by an event recorded behind it (so each figure includes what an event
    costs the queue).  Under `rocprofv3 --kernel-trace` the trace holds the
    kernels' own durations for the same launches."""
    r = Runner(torch, pkg)
    fn, _, _, keep = make_copy(r, nbytes)
    if constant_bytes:
        keep[0].fill_(3)
        fn()
    series = []
    for _ in range(bursts):
        r.tstream.synchronize()
        torch.cuda.synchronize()
        time.sleep(idle_s)
        series.append([round(x, 1) for x in r.time_each(fn, launches, 0)])
    return {"metric": "pace of back-to-back %d MiB copies of %s bytes after %.1f s idle, HIP path" % (
                nbytes // MIB, "constant" if constant_bytes else "seeded random", idle_s),
            "unit": "us per launch", "launches": launches, "pace_us": series}


# The sources that decide what the kernels do and how they are launched: the
# counter figures in profiles/hbm_traffic.json hold for one state of these.
KERNEL_SOURCES = ("blit_kernels.h", "blit_device.h", "blit_args.h", "blit_plan.h", "blit_rect.h", "blit_batch_host.h",
                  "blit_kernel_list.h")


def kernel_sources_sha256():
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "rocm-systems_amd", "csrc", name), "rb") as f:
            h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()


def load_traffic(kernel_key):
    """HBM bytes per launch from committed rocprofv3 --pmc runs (FETCH_SIZE +
    WRITE_SIZE, scaled by a plain copy kernel of known size), if recorded --
    and only if they were taken from the kernels as they are now: the file
    carries the hash of the kernel and plan sources it was measured on, and
    figures from another state of them are not reported."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        recorded = json.load(f)
    if recorded.get("kernel_sources_sha256") != kernel_sources_sha256():
        return None
    return recorded.get(kernel_key, {}).get("bytes_per_launch")


def main():
    args = parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (--gpus %d refused)" % args.gpus)
    # the clock sampler is a process of its own and is started before this one touches the GPU
    main_flow = args.workload not in ("idle_series", "sustain", "pieces", "batch_layouts", "rect_grid", "rect_check",
                                      "misaligned_classes")
    sampler = SysfsSampler(0.002).start() if main_flow and not args.no_sample else None
    import torch
    import __graft_entry__ as entry
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    pkg = entry.load_package()
    if args.workload == "idle_series":
        series = idle_series if args.path == "aql" else idle_series_hip
        print(json.dumps(series(pkg, torch, args.bytes, max(args.steps, 10), 3.0, args.constant_bytes)))
        return
    r = Runner(torch, pkg)
    nbytes = args.bytes
    if args.workload == "sustain":
        print(json.dumps(sustain_series(r)))
        r.blit.close()
        return
    if args.workload == "pieces":
        print(json.dumps({"metric": "pace of long D2D copies as one launch and cut into pieces", "unit": "us per GiB",
                          **piece_sweep(r)}))
        r.blit.close()
        return
    if args.workload == "misaligned_classes":
        print(json.dumps({"metric": "misaligned D2D copy: one offset pair per class at 1 GiB - 64 B, a length sweep at "
                                    "(3, 9), the blocking 4 KiB copy", "unit": "us per launch / GB/s",
                          "misaligned": misaligned_figures(r, pkg)}))
        r.blit.close()
        return
    if args.workload in ("rect_grid", "rect_check"):
        print(json.dumps({"metric": "region copies of whole-line rows: the plan against forced store policies and "
                                    "walk orders", "unit": "GB/s",
                          "shapes": rect_grid(r, "check" if args.workload == "rect_check" else "grid")}))
        r.blit.close()
        return
    if args.workload == "batch_layouts":
        print(json.dumps({"metric": "batched copy on several layouts", "unit": "us per batch",
                          "layouts": batch_layouts(r)}))
        r.blit.close()
        return

    if args.workload == "copy":
        fn, verify, algo, keep = make_copy(r, nbytes)
        name = "aligned D2D copy, %d MiB seeded random bytes, src/dst 256-byte aligned" % (nbytes // MIB)
        traffic_key = "copy_1GiB" if nbytes == GIB else None
    elif args.workload == "fill":
        fn, verify, algo, keep = make_fill(r, nbytes)
        name = "dword fill 0x%08X, %d MiB, 256-byte aligned" % (FILL_VALUE, nbytes // MIB)
        traffic_key = "fill_1GiB" if nbytes == GIB else None
    elif args.workload == "misaligned":
        fn, verify, algo, keep = make_copy(r, nbytes - 64, s_off=3, d_off=9)
        name = "misaligned D2D copy, %d MiB - 64 B, src&15=3 dst&15=9" % (nbytes // MIB)
        traffic_key = "misaligned_1GiB" if nbytes == GIB else None
    elif args.workload == "rect":
        shape = tuple(int(v) for v in args.rect.split(","))
        shape = shape + (0,) * (5 - len(shape))
        fn, verify, algo, keep = make_rect(r, *shape)
        name = "pitched 2-D region copy, %d rows x %d B out of %d B-pitch surfaces, x offsets %d / %d (%d MiB moved)" % (
            shape[0], shape[1], shape[2], shape[3], shape[4], shape[0] * shape[1] // MIB)
        traffic_key = "rect_%dx%d_%d" % shape[:3]
    elif args.workload == "calib":
        fn, verify, algo, keep = make_calib(r, nbytes)
        name = "calibration: torch copy_ of %d MiB (not this library)" % (nbytes // MIB)
        traffic_key = None
    else:
        fn, verify, algo, keep = make_batch(r)
        name = "65536 batched D2D copies, 64 B..256 KiB log-uniform, offsets 0..15, 16 GiB arena"
        traffic_key = "batch_65536"

    if args.tune:
        r.check(r.blit.set_tuning(**{k: int(v) for k, v in (kv.split("=") for kv in args.tune.split(","))}), "set_tuning")
        name += " [tuning: %s]" % args.tune
    # The timed region: [settle burst] [W warm-up launches] [K timed launches], back to back, and right behind
    # them the same K launches once more with an event between every two, so that the line shows launch by launch
    # what the device did around the timed region; the clocks the driver reports are sampled over all of it.
    r.tstream.synchronize()
    torch.cuda.synchronize()
    t_ready = time.perf_counter()
    t_first = time.perf_counter()
    settle_launches, settle_ms = r.settle(fn, args.settle_ms) if args.settle_ms > 0 else (0, 0.0)
    t_timed = time.perf_counter()
    wall, dev_us = r.time_launches(fn, args.steps, args.warmup)
    wall_breakdown = r.last_wall_breakdown_us
    t_replica = time.perf_counter()
    replica = r.time_each(fn, max(args.steps, 5), 0)
    t_end = time.perf_counter()
    if sampler:
        sampler.stop()
    timed_region = {
        "settle_ms": round(settle_ms, 1), "settle_launches": settle_launches,
        "host_idle_before_first_launch_ms": round((t_first - t_ready) * 1e3, 2),
        "phases_ms_since_first_launch": {"settle": [0.0, round((t_timed - t_first) * 1e3, 1)],
                                         "warmup_and_timed": [round((t_timed - t_first) * 1e3, 1),
                                                              round((t_replica - t_first) * 1e3, 1)],
                                         "one_by_one": [round((t_replica - t_first) * 1e3, 1),
                                                        round((t_end - t_first) * 1e3, 1)]},
        "us_per_launch_one_by_one": [round(u, 1) for u in replica],
        "wall_clock_us_since_timing_began": wall_breakdown,
        "sysfs_columns": (["ms since first launch"] + sampler.columns()) if sampler else None,
        "sysfs_changes": sampler.changes(t_first, t_end) if sampler else None,
        "what": "the device is brought to its sustained state by settle_ms of back-to-back launches of the workload "
                "itself (BASELINE asks for the rate a transfer sustains), then W warm-up and K timed launches follow "
                "without a gap: `value` is bytes over the host's wall clock around the K launches, roofline.kernel_us "
                "the HIP events around the same K launches.  us_per_launch_one_by_one are the next K launches, an "
                "event between every two (each figure includes the event's few microseconds of queue time).  "
                "wall_clock_us_since_timing_began says where the wall clock's microseconds beyond the device's own "
                "lie: when the host had issued the K steps, when it saw the closing event complete, when the "
                "synchronisation that closes the region had returned (the end of `value`'s clock), and the device's "
                "time between the events around the K steps",
    }
    if not args.no_verify:
        verify()
    plan = r.blit.last_plan().as_dict()
    value = algo * args.steps / wall / 1e9
    achieved = algo / dev_us / 1e3
    each = sorted(replica)
    if args.tune:
        r.blit.set_tuning()
    # and how a burst of launches runs after an idle period: 60 launches one by one after 2 s without work
    hump = hump_constant = None
    if not args.no_also:
        r.tstream.synchronize()
        time.sleep(2.0)
        hump = [round(u, 1) for u in r.time_each(fn, 60, 0)]
        hump_constant = None
        if args.workload == "copy":
            # the control: the same burst with a source of constant bytes
            const_src = r.device_bytes(nbytes + 64)
            const_src.fill_(3)
            D = aligned_ptr(keep[1])
            fn_const = lambda: r.check(r.blit.copy(D, aligned_ptr(const_src), nbytes, r.stream), "copy")
            fn_const()
            r.tstream.synchronize()
            torch.cuda.synchronize()
            time.sleep(2.0)
            hump_constant = [round(u, 1) for u in r.time_each(fn_const, 40, 0)]
            del const_src

    also = {}
    if not args.no_also:
        del keep
        torch.cuda.empty_cache()
        for key, maker in (("copy_1GiB", lambda: make_copy(r, GIB)),
                           ("fill_1GiB", lambda: make_fill(r, GIB)),
                           ("misaligned_1GiB", lambda: make_copy(r, GIB - 64, s_off=3, d_off=9)),
                           ("batch_65536", lambda: make_batch(r)),
                           ("batch_65536_device_descriptors", lambda: make_batch_device(r)),
                           ("rect_8192x131072_262144", lambda: make_rect(r))):
            f2, v2, a2, k2 = maker()
            w2, us2 = r.time_settled(f2, 30)
            v2()
            also[key] = {"gbs": round(a2 / us2 / 1e3, 1), "frac_of_peak": round(a2 / us2 / 1e3 / HBM_PEAK_GBS, 4),
                         "us_per_launch": round(us2, 2)}
            if key.startswith("batch"):
                # one batch at a time: submission to completion seen by the host
                # (us_per_launch above is the pace of batches submitted back to back)
                lat = []
                for _ in range(15):
                    t0 = time.perf_counter()
                    f2()
                    r.tstream.synchronize()
                    lat.append((time.perf_counter() - t0) * 1e6)
                also[key]["blocking_us_median"] = round(sorted(lat)[len(lat) // 2], 1)
            del f2, v2, k2
            torch.cuda.empty_cache()
        also["misaligned"] = misaligned_figures(r, pkg)
        r.torch.cuda.empty_cache()
        also["small_copy_us"] = small_copy_latency(r)
        also["size_sweep"] = size_sweep(r)
        also["rect_shapes"] = rect_shapes(r)
        r.torch.cuda.empty_cache()
        also["aql_submission"] = aql_path(r, pkg)
        also["reference_gpu_path"] = reference_gpu_path(r)
        also["host_link"] = host_link(r, pkg)

    line = {
        "metric": "D2D copy & fill GB/s (R+W) at 1 GiB on 1 MI355X",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall / args.steps * 1e3, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": name, "bytes_per_step": algo, "plan": plan,
                   "device": torch.cuda.get_device_name(0), "cus": r.blit.num_cus},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": load_traffic(traffic_key) if traffic_key else None,
                     "kernel_us": round(dev_us, 2), "algorithmic_bytes_per_launch": algo,
                     "kernel_us_median": round(each[len(each) // 2], 2), "kernel_us_best": round(each[0], 2),
                     "per_launch_note": "median and best of the %d launches timed one by one right behind the timed "
                                        "region (timed_region.us_per_launch_one_by_one; each figure includes an "
                                        "event's few microseconds of queue time; kernel_us, the mean over the "
                                        "timed region, does not)" % len(each)},
        "timed_region": timed_region,
        "idle_hump": None if hump is None else {
            "us_per_launch": hump,
            "us_per_launch_constant_bytes": hump_constant,
            "what": "60 back-to-back launches of the headline workload after 2 s without work, timed one by one "
                    "(an event between every two), and as a control 40 launches of the same copy from a source "
                    "of constant bytes (every byte 3), also after 2 s without work.  With the workload's random "
                    "bytes a burst that follows an idle period runs 4-10 % slow for some 3 ms, from about 3.5 ms "
                    "in (launches 11-20 of 1 GiB copies), on either submission path and whatever the host does "
                    "meanwhile; with constant bytes it does not, and the clocks the driver reports stay where "
                    "they are: the device's power management answering the current that toggling data draws, "
                    "not the kernel (profiles/copy_after_idle.md).  The timed region above is kept clear of that "
                    "window by its settle burst"},
        "also": also,
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(entry.load_oracle(), args.cpu_seconds)
    r.blit.close()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
