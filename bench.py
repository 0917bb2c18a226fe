"""Benchmark of the fused log-prob + entropy + PPO-loss forward+backward at V = 151936, bf16, on one MI355X.

One "step" = one pass of the hot path over one synthetic micro-batch that is already resident in HBM:
``relax_amd.policy_loss_function(args, batch, logits)`` (log-prob + entropy forward, PPO-clip 0.2/0.28 + k3 KL
coef 1e-3, token-mean aggregation) followed by ``loss.backward()`` to bf16 dlogits (for this token-local loss the
library runs both in one fused launch).  Workload = the Qwen3-8B-shaped
actor step: 16 sequences x 4096 tokens = 65536 rows x 151936 vocabulary, logits ~ N(0, 3) with 5 % spiked rows,
first 20 % of every sequence masked out.

Prints ONE JSON line (metric, value, roofline of the dominant kernel, CPU baseline of the same arithmetic).  The plain
invocation then also runs the other configurations below (up to 10 timed steps each, about a minute in all) and
reports them inside that line as ``other_workloads``; ``--no-secondary`` or ``--cpu-rows 0`` skips them.

``--workload`` selects the other configurations of the same path, each printed in the same format:
``actor_step_fp32`` (the actor step on fp32 logits [32768, 151936], the dtype stock Megatron hands a custom loss),
``cfg1`` (GRPO plumbing case: 512 responses x 256 tokens, fp32 logits [131072, 32000], rewards -> advantages -> loss),
``lmhead`` (fused LM-head + log-prob/entropy forward and dhidden/dweight backward, hidden [32768, 4096], MFMA-bound),
``reverse_kl`` (on-policy distillation, student/teacher [16384, 151936], forward + student dlogits),
``varlen_gspo`` / ``varlen_cispo`` (8 packed sequences of 2k-32k tokens, RLOO advantages, sequence-level losses),
``actor_fwd`` (the forward-only log-prob pass of the ActorFwd / Reference roles over the actor step's logits),
``actor_fwd_topk`` (the same pass with entropy and the student's top-K ids), ``actor_step_opd_topk`` (the actor step
with the top-64 on-policy-distillation term).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from types import SimpleNamespace

import torch

VOCAB = 151936
SEQS, SEQ_LEN = 16, 4096
HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
PEAK_SCLK_MHZ = 2400.0  # the shader clock the published matrix-core peak is quoted at
METRIC = "tokens/s fused logprob+entropy+loss fwd+bwd @V=151936 bf16; % HBM/MFMA peak"
PROFILES_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles")
KERNEL_CHOICE = "auto"  # --kernel-choice, as handed to relax_amd_set_kernel_choice


KNOWN_ROWS, KNOWN_VOCAB = 4099, 131072  # an odd row count no workload uses: the reference dispatches' signature
KNOWN_KIB = KNOWN_ROWS * KNOWN_VOCAB * 2 / 1024.0


def known_size_streams(dev) -> None:
    """Two untimed launches of known traffic before the timed region, the references that ``rocprofv3 --pmc
    FETCH_SIZE`` / ``WRITE_SIZE`` readings of the step's kernels are scaled by: the library's forward scan over
    4099 x 131072 bf16 logits (reads 1.0002 GiB, writes a few KB) and its row-per-workgroup backward with all-zero
    incoming gradients (such rows are zero-filled without being read: writes 1.0002 GiB, reads a few KB)."""
    from relax_amd import ops

    x = torch.ones((KNOWN_ROWS, KNOWN_VOCAB), dtype=torch.bfloat16, device=dev)
    tok = torch.zeros(KNOWN_ROWS, dtype=torch.int64, device=dev)
    zeros = torch.zeros(KNOWN_ROWS, dtype=torch.float32, device=dev)
    _, _, lse, spx = ops.logprob_entropy_fwd(x, tok, None, 1.0, True)
    prev = ops.set_kernel_choice("two_walk")
    ops.logprob_entropy_bwd(x, tok, lse, spx, zeros, zeros)
    ops.set_kernel_choice(prev)
    torch.cuda.synchronize()
    del x


def measured_traffic(kernel: str, rows: int, vocab: int):
    """(HBM bytes per launch, source file) for ``kernel`` on ``rows`` x ``vocab``, from the rocprofv3 --pmc summaries
    under profiles/: a line ``counters: kernel=<name> rows=<n> vocab=<v> FETCH_SIZE_KiB=<a> fetch_scale=<f>
    WRITE_SIZE_KiB=<b> write_scale=<g>`` gives (a * f + b * g) KiB, the per-dispatch counter readings scaled by what
    the same counters read for a plain copy of known size.  (None, None) when no summary covers this launch: the
    counters need the profiler and are not collected by this run."""
    import glob
    import re

    for path in sorted(glob.glob(os.path.join(PROFILES_DIR, "*.md"))):
        for line in open(path, errors="replace"):
            if not line.startswith("counters:"):
                continue
            m = re.match(r"counters: kernel=(.+?) rows=(\d+) vocab=(\d+) FETCH_SIZE_KiB=([\d.]+) fetch_scale=([\d.]+) "
                         r"WRITE_SIZE_KiB=([\d.]+) write_scale=([\d.]+)", line.strip())
            if m and m.group(1) == kernel and int(m.group(2)) == rows and int(m.group(3)) == vocab:
                kib = float(m.group(4)) * float(m.group(5)) + float(m.group(6)) * float(m.group(7))
                return kib * 1024.0, "profiles/" + os.path.basename(path)
    return None, None


LIVE_TRAFFIC = None  # {"fetch_KiB": {kernel: mean per dispatch}, "write_KiB": {...}, scales, command} of this run


def _pmc_pass(counter: str, argv: list, outdir: str, limit_s: int):
    """One ``rocprofv3 --pmc <counter>`` run of this file (a child process; one timed step, no CPU baseline, no other
    workloads).  Returns ([(kernel name, workgroups, counter value) per dispatch], command line) or (None, why)."""
    import csv
    import glob
    import shutil
    import subprocess

    prof = shutil.which("rocprofv3") or "/opt/rocm/bin/rocprofv3"
    if not os.path.exists(prof):
        return None, "rocprofv3 not found"
    import signal

    cmd = [prof, "--pmc", counter, "-d", outdir, "-o", "p", "--output-format", "csv", "--", sys.executable,
           os.path.abspath(__file__), *argv]
    env = dict(os.environ, TMPDIR="/tmp")
    try:
        # its own process group, so that a pass that overruns is ended together with the program it profiles
        proc = subprocess.Popen(cmd, cwd="/tmp", env=env, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True,
                                start_new_session=True)
    except OSError as e:
        return None, f"{type(e).__name__}: {e}"
    try:
        out, err = proc.communicate(timeout=limit_s)
    except subprocess.TimeoutExpired:
        try:
            os.killpg(proc.pid, signal.SIGKILL)
        except ProcessLookupError:
            pass
        proc.communicate()
        return None, f"no result within {limit_s} s"
    files = glob.glob(os.path.join(outdir, "**", "*counter_collection.csv"), recursive=True)
    if proc.returncode != 0 or not files:
        return None, f"rocprofv3 exit {proc.returncode}: {(err or out)[-300:]}"
    dispatches = []  # (kernel name, workgroups, counter value)
    with open(files[0], newline="") as f:
        for row in csv.DictReader(f):
            if row.get("Counter_Name") == counter:
                groups = int(row["Grid_Size"]) // max(1, int(row["Workgroup_Size"]))
                dispatches.append((row["Kernel_Name"], groups, float(row["Counter_Value"])))
    return dispatches, " ".join(cmd)


def collect_live_traffic(argv: list, limit_s: int = 90):
    """HBM-side bytes per launch of the step's kernels, measured in THIS run: two child runs of this file under
    ``rocprofv3 --pmc`` (FETCH_SIZE, then WRITE_SIZE: one counter per run), each scaled by what the same counter reads
    for the known-size launch the child makes before its timed step (``known_size_streams``).  Must be called before this process touches the GPU.
    Returns a dict for ``measured_traffic`` or {"error": why} (the committed summaries under profiles/ then stand in,
    and ``traffic_source`` says so)."""
    import shutil
    import tempfile

    out = {}
    tmp = tempfile.mkdtemp(prefix="relax_amd_pmc_", dir="/tmp")
    try:
        for counter, key in (("FETCH_SIZE", "fetch"), ("WRITE_SIZE", "write")):
            dispatches, info = _pmc_pass(counter, argv, os.path.join(tmp, key), limit_s)
            if dispatches is None:
                return {"error": f"{counter}: {info}"}
            ref_kernel = "logprob_entropy_fwd_kernel" if key == "fetch" else "logprob_entropy_bwd_kernel"
            known = [v for name, groups, v in dispatches if ref_kernel in name and groups == KNOWN_ROWS]
            if not known or max(known) <= 0:
                return {"error": f"{counter}: the known-size {ref_kernel} launch was not among the profiled dispatches"}
            out[key + "_scale"] = KNOWN_KIB / max(known)
            per_kernel = {}
            for name, groups, v in dispatches:
                if groups != KNOWN_ROWS:
                    per_kernel.setdefault(name, []).append(v)
            out[key + "_KiB"] = {k: sum(v) / len(v) for k, v in per_kernel.items()}
            out[key + "_command"] = info
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    return out


def live_traffic_of(kernel: str):
    """(bytes per launch, source) of ``kernel`` from this run's own counter passes, or (None, None)."""
    t = LIVE_TRAFFIC
    if not t or "error" in t:
        return None, None
    base = kernel.split("<")[0]
    want = kernel.replace(" ", "")

    def pick(table):
        exact = [v for k, v in table.items() if want in k.replace(" ", "")]
        if exact:
            return sum(exact) / len(exact)
        loose = [v for k, v in table.items() if base in k]
        return sum(loose) / len(loose) if loose else None

    f, w = pick(t["fetch_KiB"]), pick(t["write_KiB"])
    if f is None or w is None:
        return None, None
    kib = f * t["fetch_scale"] + w * t["write_scale"]
    return kib * 1024.0, (f"this run: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE child passes, per dispatch {f:.0f} x "
                          f"{t['fetch_scale']:.3f} + {w:.0f} x {t['write_scale']:.3f} KiB (scales: the same counters over known-size launches of this run)")


def assert_kernel_ran(entry: str, kernel: str) -> None:
    """The kernel names above restate the library's dispatch rule; ``relax_amd_last_kernel`` says which family the
    entry point really launched.  A disagreement would put the roofline figures under the wrong kernel's name."""
    from relax_amd import ops

    want = kernel.split("<")[0].removesuffix("_kernel")
    want = {"reverse_kl_step": "reverse_kl_step_fused"}.get(want, want)
    ran = ops.last_kernel(entry)
    assert ran == want, f"{entry} launched {ran!r}, this file expected {want!r} ({kernel})"


def hbm_roofline(kernel: str, launch_ms: float, necessary_bytes: float, rows: int, vocab: int, kernel_ms: dict,
                 ms_per_step: float, two_pass_bytes: float | None = None) -> dict:
    """Roofline block of a bandwidth-bound launch.  ``achieved`` = the bytes the launch has to move (every input row
    it needs read once, every output row written once) / its HIP-event time; ``frac`` = achieved / 8 TB/s, a true
    fraction.  ``two_pass_bytes`` (the forward-read + backward-read + write count of a two-pass implementation) is kept
    beside it as ``two_pass_*``: a kernel that keeps the row on chip moves fewer bytes than that, so the figure can
    exceed the memory system's peak and is not a roofline fraction."""
    achieved = necessary_bytes / (launch_ms * 1e-3) / 1e9
    frac = achieved / HBM_PEAK_GBS
    assert frac <= 1.0, f"roofline fraction {frac} > 1: the byte count does not describe the launch"
    traffic, source = live_traffic_of(kernel)
    if traffic is None:
        traffic, source = measured_traffic(kernel, rows, vocab)
        if traffic is not None and LIVE_TRAFFIC and "error" in LIVE_TRAFFIC:
            source += f" (committed figure; this run's counter passes failed: {LIVE_TRAFFIC['error']})"
    out = {"bound": "hbm", "kernel": kernel, "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": frac,
           "traffic": traffic, "traffic_source": source, "algorithmic_bytes_per_launch": necessary_bytes,
           "avg_launch_ms": launch_ms, "kernel_ms": kernel_ms,
           "step_GBs": necessary_bytes / (ms_per_step * 1e-3) / 1e9}
    if two_pass_bytes is not None:
        out["two_pass_bytes_per_launch"] = two_pass_bytes
        out["two_pass_GBs"] = two_pass_bytes / (launch_ms * 1e-3) / 1e9
    return out


def fused_step_kernel_name(vocab: int, dtype: str = "bf16_t") -> str:
    """Which kernel relax_amd_actor_step_fused runs for bf16 / fp32 rows of ``vocab`` entries (the library's own rule:
    one-shot workgroups sharing each row where that kernel is built; with ``--kernel-choice resident`` the persistent
    register-resident kernel in workgroups as wide as the forward-only scan's)."""
    per_vec, width, shapes = {"bf16_t": (8, 1024, ((20, False), (19, True), (18, True), (15, True), (16, False), (12, True),
                                                   (8, False), (7, True))),
                              "float": (4, 1024, ((7, True), (8, False), (12, True), (15, True), (16, False)))}[dtype]
    nvec = vocab // per_vec
    threads = 1024 if nvec >= 7168 else 512 if nvec >= 2048 else 256
    shape = (nvec // width, nvec % width != 0)
    # the one-shot kernel is built for the shapes of the persistent one and, 16-bit, for four shapes of longer rows
    split_shapes = shapes + (((24, True), (30, True), (31, True), (32, False)) if dtype == "bf16_t" else ())
    if dtype == "bf16_t" and vocab % per_vec == 0 and threads == 512 and KERNEL_CHOICE == "auto" \
            and (nvec // 512, nvec % 512 != 0) in ((7, True), (8, False), (12, True)):
        # and for 16-bit rows of 32000 / 32768 / 50304 entries, scanned by 512 virtual threads
        return f"actor_step_split_kernel<{dtype}, {nvec // 512}, {str(nvec % 512 != 0).lower()}, false, 512>"
    if vocab % per_vec == 0 and threads == width and shape in split_shapes and KERNEL_CHOICE == "auto":
        return f"actor_step_split_kernel<{dtype}, {shape[0]}, {str(shape[1]).lower()}>"
    if vocab % per_vec == 0 and threads == width and shape in shapes \
            and KERNEL_CHOICE != "two_walk":
        return f"actor_step_resident_kernel<{dtype}, {shape[0]}, {str(shape[1]).lower()}>"
    wide = ((37, True), (31, True), (32, False), (40, False), (24, True), (25, False))
    if dtype == "float" and vocab % 4 == 0 and threads == 1024 and KERNEL_CHOICE == "auto" and shape in wide + ((60, True),):
        # long fp32 rows: one-shot workgroups that keep part of their row share in LDS
        return f"actor_step_split_kernel<{dtype}, {shape[0]}, {str(shape[1]).lower()}>"
    if dtype == "float" and vocab % 4 == 0 and threads == 1024 and KERNEL_CHOICE == "resident" and shape in wide:
        # one persistent workgroup per row, the row held as its upper halves
        return f"actor_step_resident_wide_kernel<{shape[0]}, {str(shape[1]).lower()}>"
    return f"actor_step_fused_kernel<{dtype}, true, {threads}>"


def bwd_kernel_name(vocab: int) -> str:
    """Which kernel relax_amd_logprob_entropy_bwd runs for bf16 rows of ``vocab`` entries (the library's rule: one-shot
    workgroups over 4 KB chunks for rows of whole vectors; with ``--kernel-choice resident`` the persistent burst form
    for the row shapes of the register-resident step; with ``two_walk`` the row-per-workgroup loop)."""
    if KERNEL_CHOICE == "auto" and vocab % 8 == 0:
        return "logprob_entropy_bwd_chunk_kernel<bf16_t>"
    name = fused_step_kernel_name(vocab)
    if name.startswith("actor_step_resident_kernel"):
        return name.replace("actor_step_resident_kernel", "logprob_entropy_bwd_resident_kernel")
    return "logprob_entropy_bwd_kernel<bf16_t, true>"


def kl_step_kernel_name(vocab: int) -> str:
    """Which kernel relax_amd_reverse_kl_step_fused runs for bf16 rows of ``vocab`` entries (the library's rule)."""
    nvec = vocab // 8
    shape = (nvec // 1024, nvec % 1024 != 0)
    long_rows = ((20, False), (19, True), (18, True), (15, True), (16, False), (12, True))
    split_rows = long_rows + ((8, False), (7, True), (6, True), (24, True), (30, True), (31, True), (32, False))
    if vocab % 8 == 0 and KERNEL_CHOICE == "auto" and shape in split_rows:
        return f"reverse_kl_split_kernel<bf16_t, {shape[0]}, {str(shape[1]).lower()}>"
    if vocab % 8 == 0 and KERNEL_CHOICE != "two_walk" and shape in long_rows:
        return f"reverse_kl_resident_kernel<bf16_t, {shape[0]}, {str(shape[1]).lower()}>"
    return f"reverse_kl_step_kernel<bf16_t, true, {1024 if nvec >= 2048 else 256}>"


def make_args():
    return SimpleNamespace(
        advantage_estimator="grpo", eps_clip=0.2, eps_clip_high=0.28, entropy_coef=0.0, use_kl_loss=True,
        kl_loss_coef=1e-3, kl_loss_type="k3", use_unbiased_kl=False, use_rollout_logprobs=False,
        true_on_policy_mode=False, use_opsm=False, use_tis=False, get_mismatch_metrics=False,
        rollout_temperature=1.0, calculate_per_token_loss=False, qkv_format="thd", log_probs_chunk_size=-1,
        opsm_delta=1e-4, tis_clip=2.0, tis_clip_low=0.0, sapo_tau_pos=1.0, sapo_tau_neg=1.05, global_batch_size=SEQS,
    )


def make_workload(device, seqs: int, seq_len: int, vocab: int, seed: int = 0, dtype=torch.bfloat16):
    """Synthetic inputs of the named configuration, generated on the device in row blocks.  ``dtype=torch.float32``
    holds the same bf16-rounded values widened to fp32: what a bf16 output layer followed by Megatron's ``.float()``
    hands the loss hook."""
    g = torch.Generator(device=device).manual_seed(seed)
    n = seqs * seq_len
    logits = torch.empty((1, n, vocab), dtype=dtype, device=device)
    flat = logits[0]
    block = 2048
    for s in range(0, n, block):
        e = min(n, s + block)
        x = torch.randn((e - s, vocab), device=device, generator=g) * 3.0
        spike = torch.rand(e - s, device=device, generator=g) < 0.05
        cols = torch.randint(0, vocab, (e - s,), device=device, generator=g)
        x[spike, cols[spike]] += 15.0
        flat[s:e] = x.to(torch.bfloat16).to(dtype)
        del x
    tokens = [torch.randint(0, vocab, (seq_len,), device=device, generator=g) for _ in range(seqs)]
    mask = torch.ones(seq_len, device=device)
    mask[: seq_len // 5] = 0.0
    # token-mean aggregation over the micro-batch = every sample divided by the total unmasked count
    total_unmasked = float(mask.sum().item()) * seqs
    batch = dict(
        unconcat_tokens=tokens,
        total_lengths=[seq_len] * seqs,
        response_lengths=[seq_len] * seqs,  # every row is scored (response == total)
        loss_masks=[mask.clone() for _ in range(seqs)],
        advantages=[torch.randn((), device=device, generator=g).expand(seq_len).contiguous() for _ in range(seqs)],
        relax_amd_sample_denominators=torch.full((seqs,), total_unmasked, device=device),
    )
    return logits, batch, g


def attach_old_and_ref(batch, logits, args, g):
    """old = lp + N(0, 0.05), ref = lp + N(0, 0.1) around the model's own log-probs."""
    import relax_amd

    with torch.no_grad():
        _, out = relax_amd.get_log_probs_and_entropy(
            logits, args=args, unconcat_tokens=batch["unconcat_tokens"], total_lengths=batch["total_lengths"],
            response_lengths=batch["response_lengths"], with_entropy=False)
    lps = out["log_probs"]
    batch["log_probs"] = [lp + 0.05 * torch.randn(lp.shape, device=lp.device, generator=g) for lp in lps]
    batch["ref_log_probs"] = [lp + 0.1 * torch.randn(lp.shape, device=lp.device, generator=g) for lp in lps]


def cpu_baseline(args, rows: int, vocab: int, budget_s: float = 12.0, max_reps: int = 24):
    """The oracle (CPU restatement of the reference's PyTorch ops) on a bounded sample of the same workload:
    repeated fwd+bwd passes over one ``rows``-row slab until ``budget_s`` seconds of CPU work have been timed."""
    from oracle import policy as P
    from oracle import reducers as R

    threads = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
    torch.set_num_threads(threads)
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(1, rows, vocab, generator=g) * 3.0).bfloat16().float()  # the reference path receives fp32 logits
    spike = torch.rand(rows, generator=g) < 0.05
    x[0, spike, torch.randint(0, vocab, (rows,), generator=g)[spike]] += 15.0
    x.requires_grad_()
    toks = [torch.randint(0, vocab, (rows,), generator=g)]
    mask = torch.ones(rows)
    mask[: rows // 5] = 0
    base = torch.full((rows,), -12.0)
    batch = dict(unconcat_tokens=toks, total_lengths=[rows], response_lengths=[rows], loss_masks=[mask],
                 advantages=[torch.randn(rows, generator=g)], log_probs=[base], ref_log_probs=[base + 0.1])
    oargs = P.make_args(eps_clip=0.2, eps_clip_high=0.28, use_kl_loss=True, kl_loss_coef=1e-3, kl_loss_type="k3")
    red = R.make_reducer([rows], [mask])
    reps, dt = 0, 0.0
    while reps < max_reps and dt < budget_s:
        x.grad = None
        t0 = time.perf_counter()
        loss, _ = P.policy_loss_function(oargs, batch, x, red)
        loss.backward()
        dt += time.perf_counter() - t0
        reps += 1
    return {
        "value": rows * reps / dt, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"{reps} passes over {rows} rows x {vocab} vocab fp32 logits (what the reference path receives), "
                  f"fwd+bwd, {dt:.1f} s on {threads} host threads (os.cpu_count()={os.cpu_count()}); rows are "
                  f"independent, so tokens/s does not depend on the row count",
    }


class ClockSampler:
    """Samples the shader clock and the board power from sysfs while a timed region runs (a reading every 20 ms from a
    host thread; no effect on the GPU).  Matrix-core kernels on dense random operands run into the board's power limit
    and the clock drops well below the 2.4 GHz the published peak assumes, so the bench reports what it saw."""

    def __init__(self):
        import glob
        self.sclk = (glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk") or [None])[0]
        self.power = (glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input") or [None])[0]
        self.samples, self._stop, self._thread = [], False, None

    def _run(self):
        while not self._stop:
            try:
                cur = [ln for ln in open(self.sclk).read().splitlines() if "*" in ln]
                mhz = float(cur[0].split()[1].lower().replace("mhz", ""))
                watts = float(open(self.power).read()) / 1e6 if self.power else float("nan")
                self.samples.append((time.perf_counter(), mhz, watts))
            except (OSError, ValueError, IndexError):
                return
            time.sleep(0.02)

    def __enter__(self):
        if self.sclk:
            import threading
            self._thread = threading.Thread(target=self._run, daemon=True)
            self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop = True
        if self._thread:
            self._thread.join()

    def summary(self):
        """Mean over the second half of the region (the clock takes ~0.3 s to settle under load), or None."""
        if len(self.samples) < 4:
            return None
        t0, t1 = self.samples[0][0], self.samples[-1][0]
        tail = [s for s in self.samples if s[0] >= t0 + 0.5 * (t1 - t0)]
        return {"sclk_mhz": sum(s[1] for s in tail) / len(tail), "power_w": sum(s[2] for s in tail) / len(tail),
                "samples": len(tail)}


def timed_steps(step, warmup: int, steps: int):
    """``warmup`` untimed steps, then exactly ``steps`` timed ones bracketed by device synchronisation; returns
    (wall seconds, {kernel name: mean HIP-event ms per launch, launches per step}, last step's result)."""
    from relax_amd import ops

    out = None
    for _ in range(warmup):
        out = step()
    torch.cuda.synchronize()
    ops.kernel_events = []  # HIP events around the big launches, on the stream they are launched on
    t0 = time.perf_counter()
    for _ in range(steps):
        out = step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    events, ops.kernel_events = ops.kernel_events, None
    per_kernel = {}
    for name, e0, e1 in events:
        per_kernel.setdefault(name, []).append(e0.elapsed_time(e1))
    kernel_ms = {k: sum(v) / len(v) for k, v in per_kernel.items()}
    launches = {k: len(v) / steps for k, v in per_kernel.items()}
    return wall, kernel_ms, launches, out


COLLECTED = None  # a list: emit() appends its line there instead of printing it


def emit(a, n_tokens, wall, workload, config, roofline, cpu):
    out = COLLECTED.append if COLLECTED is not None else (lambda line: print(json.dumps(line)))
    out(dict({
        "metric": METRIC, "value": n_tokens / (wall / a.steps), "unit": "tokens/s", "n_gpus": 1, "steps": a.steps,
        "warmup": a.warmup, "ms_per_step": wall * 1e3 / a.steps, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": config.pop("logits_dtype", "bf16"), "data": "synthetic",
        "config": {"workload": workload, **config},
        "roofline": roofline, "cpu_baseline": cpu,
    }))


def live_rows(batch) -> int:
    """Response tokens whose loss mask is not zero: the rows a step has to read (a masked token's gradient row is
    all zeros whatever its logits hold)."""
    return int(sum(int((m != 0).sum().item()) for m in batch["loss_masks"]))


def run_actor_step(a, dev) -> None:
    import relax_amd

    args = make_args()
    args.loss_type = "policy_loss"
    fp32 = a.workload == "actor_step_fp32"
    logits, batch, g = make_workload(dev, a.seqs, a.seq_len, a.vocab, dtype=torch.float32 if fp32 else torch.bfloat16)
    attach_old_and_ref(batch, logits, args, g)
    logits.requires_grad_()
    n_tokens = a.seqs * a.seq_len
    if a.two_launch:
        args.relax_amd_single_pass = "off"
    opd = ""
    if a.opd_topk > 0:
        # on-policy distillation as production runs it: the teacher's top-K ids and log-probs of every response token,
        # reverse KL with the tail bin, added to the policy loss (opd_loss_coef)
        k = a.opd_topk
        args.opd_loss_coef, args.opd_kl_type, args.opd_token_selection = 0.5, "reverse_kl", "teacher_topk"
        args.opd_jsd_alpha, args.opd_norm_mode, args.opd_log_prob_min_clamp = 0.5, "tail", None
        args.opd_per_token_clip = args.opd_is_clip = None
        resp = batch["response_lengths"]
        batch["opd_topk_token_ids"] = [torch.randint(0, a.vocab, (r, k), device=dev, generator=g) for r in resp]
        batch["opd_topk_teacher_log_probs"] = [
            torch.log_softmax(torch.randn(r, k + 1, device=dev, generator=g), -1)[:, :k].contiguous() for r in resp]
        opd = f" + top-{k} distillation term (teacher_topk, reverse KL, tail bin)"
    # the step as the training loop runs it: loss_function applies Megatron's gradient-accumulation scaling
    # (num_microbatches / global_batch_size * dp = 1 / 16 here), so the loss's upstream gradient is not 1
    num_microbatches = 1

    def step():
        logits.grad = None
        loss, _normalizer, _log = relax_amd.loss_function(args, batch, num_microbatches, logits)
        loss.backward()
        return loss

    wall, kernel_ms, _, loss = timed_steps(step, a.warmup, a.steps)
    ms_per_step = wall * 1e3 / a.steps
    row_bytes = float(a.vocab * logits.element_size())
    live = live_rows(batch)
    # what the step must move: every live row read once, every dlogits row written once (masked rows: zeros)
    necessary = row_bytes * (live + n_tokens)
    if "actor_step_fused" in kernel_ms:
        dom, dom_name = kernel_ms["actor_step_fused"], fused_step_kernel_name(a.vocab, "float" if fp32 else "bf16_t")
        assert_kernel_ran("actor_step_fused", dom_name)
        if a.opd_topk > 0:
            dom_name = dom_name[:-1] + ", true>"  # the instantiation that evaluates the top-K term
    else:  # two launches: the backward (read live rows, write all rows) dominates; the forward read is its own launch
        dom, dom_name = kernel_ms["logprob_entropy_bwd"], bwd_kernel_name(a.vocab)
        assert_kernel_ran("logprob_entropy_bwd", dom_name)
    emit(a, n_tokens, wall,
         f"Qwen3-8B-shaped actor step: {a.seqs} seqs x {a.seq_len} tokens = {n_tokens} rows x V={a.vocab} "
         f"{'fp32 (bf16 values widened, as Megatron hands them to a custom loss)' if fp32 else 'bf16'} "
         f"logits, PPO-clip 0.2/0.28 + k3 KL 1e-3{opd}, loss_function (scale 1/{args.global_batch_size}) fwd + bwd "
         f"to dlogits",
         {"rows": n_tokens, "live_rows": live, "vocab": a.vocab, "loss": float(loss.item()),
          **({"logits_dtype": "f32"} if fp32 else {})},
         hbm_roofline(dom_name, dom, necessary, n_tokens, a.vocab, kernel_ms, ms_per_step,
                      two_pass_bytes=3.0 * row_bytes * n_tokens if "actor_step_fused" in kernel_ms else None),
         cpu_baseline(args, a.cpu_rows, a.vocab) if a.cpu_rows > 0 else None)


def run_lmhead(a, dev) -> None:
    """hidden [N, 4096] ~ N(0, 1), weight [V, 4096] ~ N(0, 0.02), scalar PPO-style loss with advantages ~ N(0, 1):
    forward log-prob + entropy without materialised logits, backward to dhidden and dweight."""
    from relax_amd.lm_head import lm_head_log_probs_and_entropy, lm_head_token_local_step

    n, h, v = a.rows or 32768, a.hidden, a.vocab
    g = torch.Generator(device=dev).manual_seed(0)
    hidden = torch.randn(n, h, device=dev, generator=g).bfloat16().requires_grad_()
    weight = (torch.randn(v, h, device=dev, generator=g) * 0.02).bfloat16().requires_grad_()
    tokens = torch.randint(0, v, (n,), device=dev, generator=g)
    adv = torch.randn(n, device=dev, generator=g) / n

    def surrogate(begin, end, lp, _ent):  # PPO's surrogate at ratio 1 (old log-probs = current ones): -A * lp
        return -(adv[begin:end] * lp).sum()

    def step():
        hidden.grad = None
        weight.grad = None
        if a.forward_only:  # the clock / power samples then belong to the forward kernel alone
            with torch.no_grad():
                lp, ent = lm_head_log_probs_and_entropy(hidden, weight, tokens, 1.0, True, False)
            return -(adv * lp).sum()
        if a.two_projections or a.keep_logits:
            # log-probs / entropy handed to autograd; backward projects again (or reads the kept logits)
            lp, ent = lm_head_log_probs_and_entropy(hidden, weight, tokens, 1.0, True, False,
                                                    keep_logits=a.keep_logits)
            loss = -(adv * lp).sum()
        else:
            # the step's default: the loss is token-local, so every slab of logits turns into its gradient as soon as
            # its log-probs are known -- one projection, a[.lmhead_slab] rows of logits in HBM at a time
            loss, lp, ent = lm_head_token_local_step(hidden, weight, tokens, surrogate, 1.0, with_entropy=True,
                                                     slab_tokens=a.lmhead_slab)
        loss.backward()
        return loss

    with ClockSampler() as clock:
        wall, kernel_ms, launches, loss = timed_steps(step, a.warmup, a.steps)
    clk = clock.summary()
    # the timed forward region holds the target-logit gather, the MFMA kernel and the split combine; the MFMA kernel
    # is > 99 % of it (see the rocprofv3 summary), so its event time stands for lmhead_fwd_kernel
    dom = kernel_ms["lmhead_logprob_fwd"]
    flops = 2.0 * n * h * v / max(launches.get("lmhead_logprob_fwd", 1.0), 1.0)  # per launch: one slab of rows
    achieved = flops / (dom * 1e-3) / 1e12
    emit(a, n, wall,
         f"fused LM-head + log-prob/entropy: hidden bf16 [{n}, {h}], weight bf16 [{v}, {h}], fwd "
         + ("(bf16 logits kept for the backward pass)" if a.keep_logits else
            "(no logits in HBM; backward projects a second time)" if a.two_projections else
            f"(logits of {min(n, a.lmhead_slab)} rows at a time become their gradient in place)")
         + (" only" if a.forward_only else " + bwd to dhidden/dweight from a scalar loss"),
         {"rows": n, "hidden": h, "vocab": v, "keep_logits": bool(a.keep_logits),
          "two_projections": bool(a.two_projections), "slab_rows": int(min(n, a.lmhead_slab)),
          "loss": float(loss.item())},
         {"bound": "mfma", "kernel": "lmhead_fwd_kernel",
          "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS,
          "unit": "TFLOP/s", "frac": achieved / MFMA_BF16_PEAK_TFLOPS, "traffic": None,
          "algorithmic_flops_per_launch": flops, "avg_launch_ms": dom, "kernel_ms": kernel_ms,
          "launches_per_step": launches,
          "step_TFLOPs_credited_6NHV": 6.0 * n * h * v / (wall / a.steps) / 1e12,
          # shader clock / board power seen during the timed steps, and the fraction of the peak rescaled to that clock
          "clock": clk, "frac_at_measured_clock":
              (achieved / (MFMA_BF16_PEAK_TFLOPS * clk["sclk_mhz"] / PEAK_SCLK_MHZ)) if clk else None},
         None)


def run_actor_fwd(a, dev) -> None:
    """The forward-only pass of the ActorFwd / Reference roles (forward_only(get_log_probs_and_entropy), with
    ``use_rollout_entropy`` off as by default): log-probs of every response row of the actor-step logits, no entropy,
    no gradient."""
    import relax_amd

    args = make_args()
    logits, batch, _ = make_workload(dev, a.seqs, a.seq_len, a.vocab)
    n_tokens = a.seqs * a.seq_len

    def step():
        with torch.no_grad():
            _, out = relax_amd.get_log_probs_and_entropy(
                logits, args=args, unconcat_tokens=batch["unconcat_tokens"], total_lengths=batch["total_lengths"],
                response_lengths=batch["response_lengths"], with_entropy=False)
        return out["log_probs"][-1][-1]

    wall, kernel_ms, _, _ = timed_steps(step, a.warmup, a.steps)
    row_bytes = float(a.vocab * logits.element_size()) * n_tokens
    emit(a, n_tokens, wall,
         f"forward-only log-probs (ActorFwd / Reference roles): {a.seqs} seqs x {a.seq_len} tokens x V={a.vocab} bf16 "
         f"logits, no entropy, no gradient",
         {"rows": n_tokens, "vocab": a.vocab},
         hbm_roofline("logprob_entropy_fwd_kernel<bf16_t, true, 1024, false>", kernel_ms["logprob_entropy_fwd"],
                      row_bytes, n_tokens, a.vocab, kernel_ms, wall * 1e3 / a.steps), None)


def run_actor_fwd_topk(a, dev) -> None:
    """The forward-only pass the actor runs when it also collects the student's top-K ids for on-policy distillation
    (compute_log_prob(collect_topk=True)): log-probs + entropy and ``topk_token_ids`` of every response row of the
    actor-step logits, no gradient."""
    import relax_amd
    from relax_amd import ops

    args = make_args()
    args.opd_log_prob_top_k = a.topk
    logits, batch, _ = make_workload(dev, a.seqs, a.seq_len, a.vocab)
    n_tokens = a.seqs * a.seq_len

    def step():
        with torch.no_grad():
            _, out = relax_amd.get_log_probs_and_entropy(
                logits, args=args, unconcat_tokens=batch["unconcat_tokens"], total_lengths=batch["total_lengths"],
                response_lengths=batch["response_lengths"], with_entropy=True, with_topk=True, topk_k=a.topk)
        return out["topk_token_ids"][-1][-1, 0].float()

    wall, kernel_ms, _, _ = timed_steps(step, a.warmup, a.steps)
    row_bytes = float(a.vocab * logits.element_size()) * n_tokens
    if "logprob_entropy_topk_fwd" in kernel_ms:
        # one read of every row serves the softmax scan and the selection (whose second, sparse look finds the row
        # in cache)
        dom, dom_name = kernel_ms["logprob_entropy_topk_fwd"], "logprob_topk_fwd_kernel<bf16_t>"
    elif "topk_rows" in kernel_ms:
        dom, dom_name = kernel_ms["topk_rows"], "topk_rows_fast_kernel<bf16_t, true>"
    else:
        dom, dom_name = kernel_ms["logprob_entropy_fwd"], "logprob_entropy_fwd_kernel<bf16_t, true, 1024>"
    emit(a, n_tokens, wall,
         f"actor forward-only pass with student top-{a.topk} ids: {a.seqs} seqs x {a.seq_len} tokens x V={a.vocab} bf16 "
         f"logits, log-prob + entropy + top-K selection",
         {"rows": n_tokens, "vocab": a.vocab, "k": a.topk},
         hbm_roofline(dom_name, dom, row_bytes, n_tokens, a.vocab, kernel_ms, wall * 1e3 / a.steps), None)


def run_reverse_kl(a, dev) -> None:
    """student / teacher bf16 logits [N, V], teacher = student + N(0, 1); per-token full-vocabulary reverse KL with a
    15 % zero loss mask, token-mean reduction, backward to the student's dlogits."""
    from relax_amd import opd_utils

    n, v = a.rows or 16384, a.vocab
    g = torch.Generator(device=dev).manual_seed(0)
    student = torch.empty((n, v), dtype=torch.bfloat16, device=dev)
    teacher = torch.empty_like(student)
    for s in range(0, n, 2048):
        e = min(n, s + 2048)
        x = torch.randn((e - s, v), device=dev, generator=g) * 3.0
        student[s:e] = x.to(torch.bfloat16)
        teacher[s:e] = (x + torch.randn((e - s, v), device=dev, generator=g)).to(torch.bfloat16)
        del x
    student.requires_grad_()
    mask = (torch.rand(n, device=dev, generator=g) >= 0.15).float()
    batch = {"loss_masks": [mask], "response_lengths": [n]}

    def step():
        student.grad = None
        if a.two_launch:
            kl = opd_utils.compute_opd_kl_full_vocab(student, teacher)
            loss = opd_utils.reduce_opd_loss(batch, kl)
        else:
            loss, _ = opd_utils.opd_loss_full_vocab(batch, student, teacher)
        loss.backward()
        return loss

    wall, kernel_ms, _, loss = timed_steps(step, a.warmup, a.steps)
    row_bytes = float(v * 2)
    if "reverse_kl_step_fused" in kernel_ms:
        # every token reports its KL, so both rows of every token are read once; one gradient row written per token
        dom, dom_name, necessary = kernel_ms["reverse_kl_step_fused"], kl_step_kernel_name(v), 3.0 * row_bytes * n
        assert_kernel_ran("reverse_kl_step_fused", dom_name)
        two_pass = 5.0 * row_bytes * n  # forward read of both rows, backward re-read of both, gradient write
    else:
        dom_name = "reverse_kl_bwd_kernel<bf16_t, true>" if KERNEL_CHOICE == "two_walk" else "reverse_kl_bwd_chunk_kernel<bf16_t>"
        dom, necessary = kernel_ms["reverse_kl_bwd"], 3.0 * row_bytes * n
        two_pass = None
    emit(a, n, wall,
         f"on-policy distillation: student/teacher bf16 logits [{n}, {v}], full-vocab reverse KL, token-mean, fwd + "
         f"student dlogits bwd",
         {"rows": n, "vocab": v, "loss": float(loss.item())},
         hbm_roofline(dom_name, dom, necessary, n, v, kernel_ms, wall * 1e3 / a.steps, two_pass_bytes=two_pass),
         None)


def run_cfg1(a, dev) -> None:
    """GRPO plumbing case: 64 prompts x group 8 = 512 responses x 256 tokens, fp32 logits [131072, 32000] ~ N(0, 2),
    rewards ~ Bernoulli(0.4), group-normalised advantages (mean / std, eps 1e-6), trailing pad of 0..63 masked tokens
    per response, PPO-clip 0.2, old = lp + N(0, 0.05), token-mean.  One step = policy loss forward + backward to fp32
    dlogits; reward post-processing + advantage broadcast run once before and are timed separately."""
    import relax_amd
    from relax_amd import utils as U

    prompts, group, resp_len, v = 64, 8, 256, 32000
    seqs = prompts * group
    n = seqs * resp_len
    cpu = torch.Generator().manual_seed(0)
    g = torch.Generator(device=dev).manual_seed(0)
    logits = torch.empty((1, n, v), dtype=torch.float32, device=dev)
    for s in range(0, n, 4096):
        logits[0, s:s + 4096] = torch.randn((min(4096, n - s), v), device=dev, generator=g) * 2.0
    rewards = torch.bernoulli(torch.full((seqs,), 0.4), generator=cpu).tolist()
    pads = torch.randint(0, 64, (seqs,), generator=cpu).tolist()
    masks = []
    for p in pads:
        m = torch.ones(resp_len, device=dev)
        if p:
            m[resp_len - p:] = 0.0
        masks.append(m)
    args = make_args()
    args.eps_clip_high = 0.2
    args.use_kl_loss = False
    args.rewards_normalization = True
    args.grpo_std_normalization = True
    args.n_samples_per_prompt = group
    args.global_batch_size = seqs
    samples = [SimpleNamespace(group_index=i // group, get_reward_value=(lambda _a, r=r: r)) for i, r in enumerate(rewards)]
    total_unmasked = float(sum(resp_len - p for p in pads))
    batch = dict(
        unconcat_tokens=[torch.randint(0, v, (resp_len,), device=dev, generator=g) for _ in range(seqs)],
        total_lengths=[resp_len] * seqs, response_lengths=[resp_len] * seqs, loss_masks=masks,
        relax_amd_sample_denominators=torch.full((seqs,), total_unmasked, device=dev),
    )
    args.use_kl_loss = False
    batch["advantages"] = [torch.zeros(resp_len, device=dev) for _ in range(seqs)]
    attach_old_and_ref(batch, logits, args, g)
    batch.pop("ref_log_probs")
    logits.requires_grad_()

    # Rewards -> group-normalised advantages happen once per rollout, not per optimisation step: timed on their own
    # (second call, warm) and reported in config.advantages_ms.
    adv_ms = 0.0
    for _ in range(2):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        _, normed = U.post_process_rewards(args, samples, device=dev)
        data = dict(log_probs=batch["log_probs"], rewards=normed, loss_masks=masks)
        relax_amd.compute_advantages_and_returns(args, data)
        torch.cuda.synchronize()
        adv_ms = (time.perf_counter() - t0) * 1e3
    batch["advantages"] = data["advantages"]

    def step():
        logits.grad = None
        loss, _ = relax_amd.policy_loss_function(args, batch, logits, None)
        loss.backward()
        return loss

    wall, kernel_ms, _, loss = timed_steps(step, a.warmup, a.steps)
    row_bytes = float(v * 4)
    dom = kernel_ms["actor_step_fused"]
    live = live_rows(batch)
    out_cpu = None
    if a.cpu_rows > 0:
        out_cpu = cpu_baseline(args, a.cpu_rows, v)
    emit(a, n, wall,
         f"GRPO plumbing: {prompts} prompts x {group} = {seqs} responses x {resp_len} tokens = {n} rows x V={v} fp32 "
         f"logits, group-normalised advantages, PPO-clip 0.2, token-mean, fwd + bwd to dlogits",
         {"rows": n, "live_rows": live, "vocab": v, "loss": float(loss.item()), "logits_dtype": "f32",
          "advantages_ms": adv_ms},
         hbm_roofline(fused_step_kernel_name(v, "float"), dom, row_bytes * (live + n), n, v, kernel_ms,
                      wall * 1e3 / a.steps, two_pass_bytes=3.0 * row_bytes * n),
         out_cpu)


def run_varlen(a, dev, loss_kind: str) -> None:
    """8 packed sequences with lengths ~ U[2k, 32k], 3-6 masked tool-output spans (~30 % of tokens) per sequence,
    RLOO advantages from rewards ~ U[0, 1] over the group of 8, GSPO (clip 3e-4/4e-4) or CISPO loss,
    sequence-mean-token-sum aggregation."""
    import relax_amd
    from relax_amd import ppo_utils

    cpu = torch.Generator().manual_seed(0)
    seqs, v = 8, a.vocab
    lengths = [int(x) for x in torch.randint(2048, 32769, (seqs,), generator=cpu)]
    while sum(lengths) > 131072:
        lengths[lengths.index(max(lengths))] //= 2
    n = sum(lengths)
    g = torch.Generator(device=dev).manual_seed(0)
    logits = torch.empty((1, n, v), dtype=torch.bfloat16, device=dev)
    for s in range(0, n, 2048):
        e = min(n, s + 2048)
        logits[0, s:e] = (torch.randn((e - s, v), device=dev, generator=g) * 3.0).to(torch.bfloat16)
    masks = []
    for ln in lengths:
        m = torch.ones(ln)
        spans = int(torch.randint(3, 7, (1,), generator=cpu))
        for _ in range(spans):
            w = int(0.3 * ln / spans)
            st = int(torch.randint(0, ln - w, (1,), generator=cpu))
            m[st:st + w] = 0.0
        masks.append(m.to(dev))
    args = make_args()
    args.advantage_estimator = loss_kind
    args.use_kl_loss = False
    if loss_kind == "gspo":
        args.eps_clip, args.eps_clip_high = 3e-4, 4e-4
    rewards = torch.rand(seqs, generator=cpu).to(dev)
    shaped = ppo_utils.compute_rloo_leave_one_out_rewards(rewards)
    batch = dict(
        unconcat_tokens=[torch.randint(0, v, (ln,), device=dev, generator=g) for ln in lengths],
        total_lengths=lengths, response_lengths=lengths, loss_masks=masks,
        advantages=[shaped[i].expand(ln).contiguous() for i, ln in enumerate(lengths)],
    )
    # sequence-mean-token-sum aggregation of pg_loss through the reference's own reducer hook (loss.py:1062-1072):
    # every sample's masked token sum divided by the number of sequences; the returned reducer carries its divisors,
    # so the step stays on the fused launches
    args.custom_pg_loss_reducer_function_path = "relax_amd.cp_utils.get_seq_mean_token_sum_reducer"
    attach_old_and_ref(batch, logits, args, g)
    logits.requires_grad_()

    def step():
        logits.grad = None
        loss, _ = relax_amd.policy_loss_function(args, batch, logits, None)
        loss.backward()
        return loss

    wall, kernel_ms, _, loss = timed_steps(step, a.warmup, a.steps)
    row_bytes = float(v * 2)
    live = live_rows(batch)
    fused = "actor_step_fused" in kernel_ms
    name = "actor_step_fused" if fused else "logprob_entropy_bwd"
    dom = kernel_ms[name]
    read_rows = live
    if not fused:
        # the separate backward launch knows every token's gradient coefficients before it starts and reads only the
        # rows whose coefficients are not both zero (GSPO: every token of a sequence whose ratio is clipped has none)
        read_rows = sum(int((logits.grad[0, s0:s0 + 4096] != 0).any(dim=1).sum().item()) for s0 in range(0, n, 4096))
    emit(a, n, wall,
         f"packed varlen: {seqs} sequences {lengths} = {n} rows x V={v} bf16 logits, ~30 % masked spans, RLOO "
         f"advantages, {loss_kind.upper()} loss, sequence-mean-token-sum, fwd + bwd to dlogits",
         {"rows": n, "live_rows": live, "rows_read_by_the_launch": read_rows, "vocab": v, "loss": float(loss.item()),
          "lengths": lengths},
         hbm_roofline(fused_step_kernel_name(v) if fused else bwd_kernel_name(v), dom,
                      row_bytes * (read_rows + n), n, v, kernel_ms, wall * 1e3 / a.steps,
                      two_pass_bytes=3.0 * row_bytes * n if fused else None),
         None)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="actor_step",
                    choices=["actor_step", "actor_step_opd_topk", "actor_step_fp32", "cfg1", "lmhead", "reverse_kl", "varlen_gspo",
                             "varlen_cispo", "actor_fwd", "actor_fwd_topk"])
    ap.add_argument("--seqs", type=int, default=SEQS)
    ap.add_argument("--seq-len", type=int, default=SEQ_LEN)
    ap.add_argument("--vocab", type=int, default=VOCAB)
    ap.add_argument("--rows", type=int, default=0, help="token rows of the lmhead / reverse_kl workloads (0 = default)")
    ap.add_argument("--hidden", type=int, default=4096, help="hidden size of the lmhead workload")
    ap.add_argument("--cpu-rows", type=int, default=2048, help="rows of the CPU baseline slab (0 = skip)")
    ap.add_argument("--keep-logits", action="store_true",
                    help="lmhead workload: keep a [V, N] bf16 copy of the logits for the backward pass instead of "
                         "projecting a second time (10 GB at the default size)")
    ap.add_argument("--two-projections", action="store_true",
                    help="lmhead: log-probs handed to autograd, the backward pass recomputes the projection")
    ap.add_argument("--lmhead-slab", type=int, default=8192,
                    help="lmhead: rows of logits that exist in HBM at a time in the one-projection step")
    ap.add_argument("--forward-only", action="store_true",
                    help="lmhead workload: time the forward pass alone (clock samples of that kernel only)")
    ap.add_argument("--topk", type=int, default=64, help="k of the actor_fwd_topk workload")
    ap.add_argument("--two-launch", action="store_true",
                    help="use the separate forward / backward launches (the path GSPO takes) instead of the fused step")
    ap.add_argument("--opd-topk", type=int, default=0,
                    help="actor_step: add the top-K on-policy distillation term with this K (0 = none)")
    ap.add_argument("--no-secondary", action="store_true",
                    help="plain invocation only: skip the other configurations that otherwise run after the headline "
                         "workload and ride along in its line as other_workloads")
    ap.add_argument("--traffic", choices=["auto", "live", "off"], default="auto",
                    help="roofline.traffic: 'live' measures it in this run (two child runs of this file under "
                         "rocprofv3 --pmc before the timed steps, about a minute); 'off' takes the figure committed "
                         "under profiles/; 'auto' = live for the plain invocation, off otherwise")
    ap.add_argument("--kernel-choice", choices=["auto", "two_walk", "resident"], default="auto",
                    help="relax_amd_set_kernel_choice: which of the two bit-identical kernels the fused entry points "
                         "launch (two_walk = the row-per-workgroup kernels for every row length)")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (token rows shard without any exchange). "
              "Run with --gpus 1.", file=sys.stderr)
        return 2
    plain = a.workload == "actor_step" and a.opd_topk == 0 and a.cpu_rows > 0 and not a.no_secondary
    if a.traffic == "live" or (a.traffic == "auto" and plain):
        # before anything in this process touches the GPU: the children are separate programs under the profiler
        global LIVE_TRAFFIC

        def child_args(workload):
            child = ["--workload", workload, "--steps", "1", "--warmup", "1", "--cpu-rows", "0", "--no-secondary",
                     "--traffic", "off", "--seqs", str(a.seqs), "--seq-len", str(a.seq_len), "--vocab", str(a.vocab),
                     "--kernel-choice", a.kernel_choice]
            if a.rows:
                child += ["--rows", str(a.rows)]
            if a.two_launch:
                child.append("--two-launch")
            if a.opd_topk and workload == a.workload:
                child += ["--opd-topk", str(a.opd_topk)]
            return child

        LIVE_TRAFFIC = collect_live_traffic(child_args(a.workload))
        if plain and "error" not in LIVE_TRAFFIC:
            # the bandwidth-bound configurations that ride along get their own counter passes (a few seconds each);
            # the first pass that fails ends the series, so a box without a working profiler costs one time limit
            for name in SECONDARY:
                if name != "lmhead":
                    SECONDARY_TRAFFIC[name] = collect_live_traffic(child_args(name))
                    if "error" in SECONDARY_TRAFFIC[name]:
                        break
    if not torch.cuda.is_available():
        print("bench.py needs a ROCm GPU", file=sys.stderr)
        return 2
    import relax_amd  # noqa: F401  (fails loudly when the HIP library is missing)
    from relax_amd import ops

    global KERNEL_CHOICE
    KERNEL_CHOICE = a.kernel_choice
    ops.set_kernel_choice(a.kernel_choice)

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    known_size_streams(dev)
    if a.workload == "actor_step_opd_topk" and a.opd_topk == 0:
        a.opd_topk = 64
    if a.workload == "actor_step_fp32" and a.seqs == SEQS:
        a.seqs = SEQS // 2  # 32768 rows: the same 19.9 GB of logits as the bf16 step
    if a.opd_topk > 0:
        a.cpu_rows = 0  # the CPU baseline is timed on the headline workload only
    if a.workload == "actor_step" and a.opd_topk == 0 and a.cpu_rows > 0 and not a.no_secondary:
        return run_default_with_secondary(a, dev)
    run_workload(a, dev)
    return 0


def run_workload(a, dev) -> None:
    if a.workload in ("actor_step", "actor_step_opd_topk", "actor_step_fp32"):
        run_actor_step(a, dev)
    elif a.workload == "cfg1":
        run_cfg1(a, dev)
    elif a.workload == "lmhead":
        run_lmhead(a, dev)
    elif a.workload == "reverse_kl":
        run_reverse_kl(a, dev)
    elif a.workload == "actor_fwd":
        run_actor_fwd(a, dev)
    elif a.workload == "actor_fwd_topk":
        run_actor_fwd_topk(a, dev)
    else:
        run_varlen(a, dev, a.workload.split("_")[1])


SECONDARY_TRAFFIC = {}  # workload -> collect_live_traffic() result, filled by the plain invocation before it touches the GPU
SECONDARY = ("lmhead", "reverse_kl", "varlen_gspo", "varlen_cispo", "cfg1", "actor_fwd", "actor_fwd_topk",
             "actor_step_opd_topk", "actor_step_fp32")


def run_default_with_secondary(a, dev) -> int:
    """The plain invocation (no ``--workload``, CPU baseline on): the headline workload exactly as ``--workload
    actor_step`` measures it, and after it the other configurations of the path with at most 10 timed steps each, so
    that one run of this file on one box covers them all.  Their figures ride along in the headline line as
    ``other_workloads`` (a few figures of each workload's own line, kept short: ``ms_per_step``, ``tokens_per_s``, the
    dominant kernel with its launch time and roofline fraction); they take some ten seconds and change nothing in the
    headline measurement, which is finished before they start."""
    import copy
    import gc

    global COLLECTED, LIVE_TRAFFIC
    COLLECTED = []
    run_actor_step(a, dev)
    line = COLLECTED.pop()
    others = {}
    for name in SECONDARY:
        LIVE_TRAFFIC = SECONDARY_TRAFFIC.get(name)
        gc.collect()
        torch.cuda.empty_cache()
        b = copy.copy(a)
        b.workload, b.steps, b.warmup, b.cpu_rows, b.rows = name, min(a.steps, 10), min(a.warmup, 3), 0, 0
        b.opd_topk = 64 if name == "actor_step_opd_topk" else 0
        if name == "actor_step_fp32":
            b.seqs = max(1, a.seqs // 2)  # half the rows: the same 19.9 GB of logits as the bf16 step
        b.traffic = "off"
        try:
            run_workload(b, dev)
            got = COLLECTED.pop()
            r = got["roofline"]
            others[name] = {"ms_per_step": round(got["ms_per_step"], 4), "tokens_per_s": round(got["value"]),
                            "steps": got["steps"], "kernel": r["kernel"], "bound": r["bound"],
                            "avg_launch_ms": round(r["avg_launch_ms"], 4), "achieved": round(r["achieved"], 1),
                            "unit": r["unit"], "frac": round(r["frac"], 4)}
            if r.get("traffic"):
                others[name]["traffic"] = round(r["traffic"])
                others[name]["traffic_over_algorithmic"] = round(r["traffic"] / r["algorithmic_bytes_per_launch"], 3)
                others[name]["traffic_measured_in_this_run"] = r["traffic_source"].startswith("this run")
        except Exception as e:  # a secondary workload must not cost the headline line
            others[name] = {"error": f"{type(e).__name__}: {e}"}
            COLLECTED.clear()
    COLLECTED = None
    line["other_workloads"] = others
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
