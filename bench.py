#!/usr/bin/env python3
"""Benchmark of the GLIF3 hot path on one MI355X.

Workload (N=1): the V1-scale forward simulation -- 230,924 GLIF3 neurons in 111
parameter classes, lognormal in-degree with mean 300 (~70 M recurrent
synapses), 17,400 Poisson inputs at 5 Hz through ~8 M input synapses, 4
receptors, delays 1-5 steps, dt = 1 ms, batch 1, 3000 simulation steps.

One "step" of this benchmark (--steps K, --warmup W) is one PASS of the hot
path over that workload: one call of the forward simulation over 3000
simulation steps of 1 ms, i.e. what one ``nest.Simulate(3000.0)`` is for the
reference (bmtk/simulator/pointnet/pointsimulator.py:159-166).  Before the
warm-up passes the network runs untimed until it has left the transient from
rest (at least 400 steps), so every timed pass sees the settled activity
(~2.8 Hz, ~230 k synaptic events per simulation step) whatever K and W are.
Recurrent weights are lognormal(0,1) pA signed by the source class as
specified; input weights are scaled by 7 because at 1 pA the network stays
silent and there would be no synaptic events to count.

Prints ONE JSON line: value = neuron-updates/s of the whole job; synaptic
events/s, the roofline of the dominant kernel, the isolated state-update and
propagation kernels, and the CPU baseline ride along in the same object.
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E bandwidth
B_PER_UPDATE_CLASS = 103       # 12 state words in + 12 out, 4 B current, 1 B flag, 2 B class id
B_PER_UPDATE_PLAIN = 101       # same without the class id
B_PER_EVENT = 18               # 4 index + 4 weight + 1 delay + 1 receptor + 8 ring read-modify-write

N_V1, N_IN, MEAN_IN, N_IN_SYN, N_CLASSES = 230924, 17400, 300, 8_000_000, 111
IN_RATE_HZ, IN_W_SCALE = 5.0, 7.0
SIM_STEPS = 3000               # simulation steps of one pass (the configuration's run length)
SETTLE_STEPS, SETTLE_MAX_STEPS = 400, 2000
CPU_MIN_STEPS = 200


def profile_traffic(file_name, key):
    """HBM bytes from a committed rocprofv3 counter summary: the value of the line ``TRAFFIC <key> = <number>``
    in profiles/<file_name> (written there from the FETCH_SIZE / WRITE_SIZE runs the file describes), or None
    when the file or the line is missing.  These are constants of those profile runs; this script does not
    re-measure them."""
    try:
        txt = open(os.path.join(ROOT, "profiles", file_name)).read()
    except OSError:
        return None
    m = re.search(r"^TRAFFIC\s+%s\s*=\s*([0-9.eE+-]+)" % re.escape(key), txt, flags=re.M)
    return float(m.group(1)) if m else None


def build_v1(torch, steps_total, resident="auto", in_w_scale=IN_W_SCALE):
    import numpy as np
    from bmtk_amd import ops, synthetic
    from bmtk_amd.simulator import Glif3Simulator
    rng = np.random.default_rng(3)
    par = synthetic.random_cells(rng, N_CLASSES)
    class_id = rng.integers(0, N_CLASSES, N_V1).astype(np.int32)
    by_tgt, by_src, _ = synthetic.device_network(N_V1, MEAN_IN, "lognormal", seed=3)
    del by_tgt
    inp = synthetic.device_input_table(N_IN, N_V1, N_IN_SYN, seed=4, w_scale=in_w_scale)
    # exponential inter-spike intervals per source, generated on the device (ops.poisson_events)
    in_ptr, in_ev = ops.poisson_events(N_IN, IN_RATE_HZ, 1.0, steps_total, seed=5)
    sim = Glif3Simulator(N_V1, par, 1.0, class_id=class_id, rec=by_src, inp=inp, resident=resident)
    sim.set_input_events(in_ptr, in_ev)
    return sim, par, class_id


def count_events(torch, sim, bits, step0):
    """Synaptic events caused by the spikes in `bits` and by the input events of the same steps."""
    rec = sim.synaptic_events(bits)
    k0, k1 = int(sim.in_ptr[step0].item()), int(sim.in_ptr[step0 + bits.shape[0]].item())
    ev = sim.in_events[k0:k1].long() // sim.batch
    deg = (sim.inp.indptr[1:] - sim.inp.indptr[:-1]).long()
    return rec, int(deg[ev].sum().item())


def time_region(torch, fn):
    """(wall seconds, HIP-event seconds on the current stream) around fn()."""
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    fn()
    e1.record()
    torch.cuda.synchronize()
    return time.perf_counter() - t0, e0.elapsed_time(e1) * 1e-3


def bench_state_update(torch, steps=1000, warmup=50):
    """Isolated fused state update: N = 1,048,576, Gaussian(0, 50 pA) currents from a pool of 8 pre-generated
    vectors, in two forms: parameters from a table of 111 classes (the form the V1-scale simulation uses:
    101 B of state, current and flag plus the 2 B class id per update) and per-neuron parameters (29
    propagator words more per update)."""
    import numpy as np
    from bmtk_amd import ops, synthetic
    n = 1 << 20
    out = []
    for form in ("class table", "per-neuron parameters"):
        rng = np.random.default_rng(1)
        if form == "class table":
            par = synthetic.random_cells(rng, N_CLASSES)
            cid_h = rng.integers(0, N_CLASSES, n).astype(np.int32)
            cid = torch.as_tensor(cid_h, device="cuda")
            per_update = B_PER_UPDATE_CLASS
            key = "hbm_bytes_per_launch_class_table"
        else:
            par = synthetic.random_cells(rng, n)
            cid_h = cid = None
            per_update = B_PER_UPDATE_PLAIN + 29 * 4
            key = "hbm_bytes_per_launch"
        prop = ops.glif3_precompute(par, 1.0)
        st = ops.Glif3State.from_numpy(synthetic.random_state(rng, par, n, 1, class_id=cid_h))
        pool = [torch.randn(n, device="cuda") * 50.0 for _ in range(8)]
        z = torch.zeros(n, dtype=torch.uint8, device="cuda")
        for k in range(warmup):
            ops.glif3_step_fwd(st, prop, 1.0, class_id=cid, i_ext=pool[k % 8], z=z)
        wall, dev = time_region(torch, lambda: [ops.glif3_step_fwd(st, prop, 1.0, class_id=cid, i_ext=pool[k % 8], z=z)
                                                for k in range(steps)])
        per = dev / steps
        alg = n * per_update
        out.append({"kernel": "glif3_step_kernel", "workload": "state update N=1048576, %s, %d steps" % (form, steps),
                    "neuron_updates_per_s": n / per, "us_per_launch": per * 1e6,
                    "roofline": {"bound": "hbm", "achieved": alg / per / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                 "frac": alg / per / 1e9 / HBM_PEAK_GBS,
                                 "traffic": profile_traffic("glif3_step_kernel_state_update_1M.txt", key)},
                    "bytes_per_update": per_update})
    return out


def bench_compaction(torch, steps=200, warmup=20):
    """Spike compaction at the propagation workload's size: 51,978 neurons x 64 trials = 3.3 M elements at
    5 Hz x 1 ms, from byte flags and from spike-bit words.  Algorithmic bytes: the scan reads 1 B (1 bit) per
    element and writes 4 B per spike."""
    from bmtk_amd import ops
    n = 51978 * 64
    g = torch.Generator(device="cuda").manual_seed(7)
    z = (torch.rand(n, device="cuda", generator=g) < 5e-3).to(torch.uint8)
    words = (n + 63) // 64
    pad = torch.zeros(words * 64, dtype=torch.uint8, device="cuda")
    pad[:n] = z
    weights = (2 ** torch.arange(64, device="cuda", dtype=torch.int64))
    bits = (pad.view(words, 64).to(torch.int64) * weights).sum(1)  # bit 63 wraps into the sign: intended
    bits = torch.cat([bits, bits.new_zeros(1)])
    comp = ops.SpikeCompactor(n)
    out = []
    for name, src, scan_bytes in (("flags", z, n), ("bits", bits, n // 8)):
        for _ in range(warmup):
            comp(src)
        wall, dev = time_region(torch, lambda: [comp(src) for _ in range(steps)])
        per = dev / steps
        count = int(comp.count.item())
        alg = scan_bytes + 4 * count
        out.append({"kernel": "compact_count + compact_write_fused (%s)" % name,
                    "workload": "compaction of %d elements, %d spikes" % (n, count),
                    "elements_per_s": n / per, "us_per_call": per * 1e6,
                    "roofline": {"bound": "hbm", "achieved": alg / per / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                 "frac": alg / per / 1e9 / HBM_PEAK_GBS, "traffic": None}})
    return out


PROPAGATION_MODES = ("scatter", "gather", "pull", "pull2", "auto", "auto2")
PROPAGATION_RATES = (0.2, 1.0, 5.0, 20.0)


def bench_propagation(torch, steps=200, warmup=20, modes=PROPAGATION_MODES, rates=PROPAGATION_RATES):
    """Isolated spike propagation: 51,978 neurons, Poisson(1000) in-degree
    (~52 M synapses), batch 64, Bernoulli spikes at 0.2, 1, 5 and 20 Hz.  Six forms: the event-driven scatter, the
    row-wise gather, the pull over the spike history of the last L steps, the same pull for two arrival steps per
    pass over the table (`pull2`, timed per arrival step), `auto`, which decides on the device,
    step by step, between pushing a step's spikes as events and leaving them to the pull, and `auto2`, the same
    switch called every second step with the two-step pull behind it (timed per arrival step).  A pool of L spike
    patterns serves as the history (row k % L = the spikes of step k)."""
    from bmtk_amd import ops, synthetic
    n, batch, L = 51978, 64, 6
    by_tgt, by_src, _ = synthetic.device_network(n, 1000, "poisson", seed=2)
    t_tgt = ops.SynapseTable.from_device(by_tgt, n, n, L)
    t_src = ops.SynapseTable.from_device(by_src, n, n, L)
    ne = n * batch
    ring = torch.zeros(L, 4, ne, device="cuda")
    comp = ops.SpikeCompactor(ne)
    deg = (t_src.indptr[1:] - t_src.indptr[:-1]).long()
    out = []
    g = torch.Generator(device="cuda")
    g.manual_seed(7)
    for rate in rates:
        pool_bits, pool_ev = [], []
        for _ in range(L):
            z = (torch.rand(ne, device="cuda", generator=g) < rate * 1e-3)
            zb = torch.zeros(ops.n_words(ne) + 1, dtype=torch.int64, device="cuda")
            ids, count = comp(z.to(torch.uint8))
            c = int(count.item())
            pool_ev.append((ids[:c].clone(), count.clone(), int(deg[(ids[:c].long() // batch)].sum().item())))
            # spike bits of the same flags
            w = z.view(-1, 64).to(torch.int64)
            zb[:-1] = (w << torch.arange(64, device="cuda")).sum(1)
            pool_bits.append(zb)
        events = sum(e for _, _, e in pool_ev) / len(pool_ev)
        active = sum(int(c.item()) for _, c, _ in pool_ev) / len(pool_ev)
        hist = torch.stack(pool_bits)                              # spike bits of the last L steps
        syn = torch.zeros(4, ne, device="cuda")
        syn2 = torch.zeros(2, 4, ne, device="cuda")
        auto = ops.AutoPropagator(t_src, t_tgt, hist, ring, n, n, batch)
        auto2 = ops.AutoPropagator2(t_src, t_tgt, hist, ring, n, n, batch)
        for mode in modes:
            def one(k):
                if mode == "scatter":
                    ids, count, _ = pool_ev[k % L]
                    ops.csr_propagate_scatter(ids, count, t_src, ring, n, batch, k)
                elif mode == "auto":
                    ids, count, _ = pool_ev[k % L]
                    auto.step(k, ids, count)
                elif mode == "gather":
                    ops.csr_propagate_gather(pool_bits[k % L], n, t_tgt, ring, n, batch, k)
                elif mode == "pull2":                                  # two arrival steps per call, every other step
                    if k % 2 == 0:
                        ops.csr_propagate_pull2(hist, n, t_tgt, syn2, n, batch, k + L + 1)
                elif mode == "auto2":                                  # likewise: the two-step form of the switch
                    if k % 2 == 1:
                        auto2.step2(k, pool_ev[(k - 1) % L][0], pool_ev[(k - 1) % L][1], pool_ev[k % L][0], pool_ev[k % L][1])
                else:
                    ops.csr_propagate_pull(hist, n, t_tgt, syn, n, batch, k + L)
            for k in range(warmup):
                one(k)
            ring.zero_()
            wall, dev = time_region(torch, lambda: [one(k) for k in range(warmup, warmup + steps)])
            per = dev / steps
            alg = events * B_PER_EVENT
            traffic = profile_traffic("propagation_kernels_52k_batch64.txt", "hbm_bytes_per_launch_%s_%gHz" % (mode, rate))
            two = mode in ("pull2", "auto2")
            if traffic is not None and two:
                traffic /= 2                                            # per arrival step, like the time below
            entry = {"kernel": {"auto": "auto_push_kernel or pull_kernel, chosen on the device",
                                "auto2": "auto2: auto_push_kernel or pull2_kernel, chosen on the device for each of the two steps of a call",
                                "pull2": "pull2_kernel: the arrivals of two steps per launch, half a launch per step"}
                               .get(mode, mode + "_kernel"),
                     "workload": "propagation N=51978 nnz=%d batch=64 rate=%gHz" % (t_src.nnz, rate),
                     "events_per_launch": events, "active_elements_per_launch": active,
                     "synaptic_events_per_s": events / per, "us_per_launch": per * 1e6 * (2 if two else 1),
                     "us_per_arrival_step": per * 1e6,
                     "roofline": {"bound": "hbm", "achieved": alg / per / 1e9, "peak": HBM_PEAK_GBS,
                                  "unit": "GB/s", "frac": alg / per / 1e9 / HBM_PEAK_GBS, "traffic": traffic,
                                  "hbm_frac": None if traffic is None else traffic / per / 1e9 / HBM_PEAK_GBS}}
            if mode in ("auto", "auto2"):
                which = auto if mode == "auto" else auto2
                entry["pulled"] = bool(which.pulled_steps().any())
                entry["scatter_max_active"] = which.scatter_max_active
            out.append(entry)
    return out


def bench_bptt(torch, steps=600):
    """One BPTT training step: 51,978 neurons (Poisson in-degree 1000, ~52 M synapses) plus 17,400
    Poisson inputs at 5 Hz, batch 32, 600 steps; triangular surrogate (dampening 0.3); MSE between
    the rates of 17 random populations and random targets; gradients for every recurrent and input
    weight.  Recurrent weights are scaled by 0.2 and input weights by 2 so that the network settles
    near 3 Hz (unit weights at this in-degree saturate it).

    Returns three entries: the training step, and the transposed propagation on its own (the kernel that
    takes most of the backward pass) in the two forms the library has: through the table regrouped by target
    range (bmtk_csr_propagate_bwd_blocked, the form the training step uses at this size) and row by row through
    the source-major table (bmtk_csr_propagate_bwd).
    Rooflines use the bytes that MUST cross HBM: per backward step the packed table once (8 B per synapse),
    the adjoint ring slots once (L-1 slots x 4 receptors x ne x 4 B), the adjoint state in and out, the
    forward record (potential and flags) and the input gradient's reads; not the L2 fills the kernels cause by
    fetching an adjoint row per synapse (those are in `traffic`)."""
    import numpy as np
    from bmtk_amd import ops, synthetic, training
    from bmtk_amd.simulator import Glif3Simulator
    n, n_in, batch = 51978, 17400, 32
    rng = np.random.default_rng(4)
    par = synthetic.random_cells(rng, n)
    _, by_src, _ = synthetic.device_network(n, 1000, "poisson", seed=2, w_scale=0.2)
    inp = synthetic.device_input_table(n_in, n, 8_000_000, seed=4, w_scale=2.0)
    in_ptr, in_ev = ops.poisson_events(n_in, 5.0, 1.0, 2 * steps, batch=batch, seed=5)
    sim = Glif3Simulator(n, par, 1.0, batch=batch, rec=by_src, inp=inp, resident=False)
    sim.set_input_events(in_ptr, in_ev)
    g = torch.Generator(device="cuda").manual_seed(11)
    pop = torch.randint(0, 17, (n,), device="cuda", generator=g)
    targets = torch.rand(batch, 17, device="cuda", generator=g) * 0.01
    bptt = training.Glif3Bptt(sim, dampening=0.3)
    res = {}

    def fwd():
        res["fwd"] = sim.run(steps, save_state=True)

    def bwd():
        counts = training.spike_counts(res["fwd"]["bits"], sim.ne)
        res["loss"], g = training.rate_mse(counts, steps, batch, pop, targets)
        res["counts"] = counts
        bptt.zero()
        bptt.backward(res["fwd"], dl_dz_const=g)

    fwd(); bwd()                              # warm-up step (also leaves the transient from rest behind)
    t_f, _ = time_region(torch, fwd)
    t_b, _ = time_region(torch, bwd)
    deg = (sim.rec.indptr[1:] - sim.rec.indptr[:-1]).long()
    spikes = res["counts"].view(n, batch).sum(1)
    events = int((spikes.long() * deg).sum().item())
    ne, L, nnz, nnz_in = sim.ne, sim.L, sim.rec.nnz, sim.inp.nnz
    ring_bytes = (L - 1) * 4 * ne * 4
    # backward, per step: table + adjoint slots (transposed propagation), 11 adjoint state words in and out + the
    # new slot out + potential and flags in (state adjoint), the input table rows of the step's events
    bwd_step = nnz * 8 + ring_bytes + ne * (11 * 8 + 16 + 5) + (in_ev.numel() / (2 * steps)) * (nnz_in / n_in) * 8
    # forward, per step: the joint target-major table once (recurrent and input synapses, 8 B each), 12 state words
    # in and out, the record (potential and flags) out, the neuron's propagator column once per neuron
    fwd_step = (nnz + nnz_in) * 8 + ne * (12 * 8 + 5) + n * 29 * 4
    step_entry = {
        "kernel": "%s (forward), bwd_gather_blocked2_kernel + bwd_state2_kernel (backward, two steps per launch; both "
                  "weight gradients ride in the former)" %
                  ("sim_fused_kernel: pull and update fused, two steps per launch" if sim.fuse_table is not None
                   else "sim_step_kernel + pull_kernel"),
        "blocked_table_ranges": bptt.n_blocks if bptt.blk is not None else 0,
        "workload": "BPTT step N=51978 nnz=%d inputs=17400 batch=32 steps=%d" % (nnz, steps),
        "seconds_per_training_step": t_f + t_b, "forward_s": t_f, "backward_s": t_b,
        "mean_rate_hz": float(res["counts"].float().mean().item()) / steps * 1e3,
        "recurrent_events_forward": events, "loss": float(res["loss"]),
        "weight_grad_events_per_s": events / t_b,
        "grad_norm_rec": float(bptt.d_rec_w.norm().item()), "grad_norm_inp": float(bptt.d_inp_w.norm().item()),
        "roofline": {"bound": "hbm", "achieved": bwd_step * steps / t_b / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": bwd_step * steps / t_b / 1e9 / HBM_PEAK_GBS, "what": "backward pass, HBM-compulsory bytes",
                     "algorithmic_bytes_per_step": bwd_step,
                     "traffic": profile_traffic("training_step_kernels_52k_batch32.txt", "hbm_bytes_per_backward_step")},
        "roofline_forward": {"bound": "hbm", "achieved": fwd_step * steps / t_f / 1e9, "peak": HBM_PEAK_GBS,
                             "unit": "GB/s", "frac": fwd_step * steps / t_f / 1e9 / HBM_PEAK_GBS,
                             "algorithmic_bytes_per_step": fwd_step,
                             "what": "the joint table once per step + state in and out + record out (the kernel reads "
                                     "the table once per TWO steps, so its traffic is below this)",
                             "frac_by_update_and_event_bytes":
                                 (ne * B_PER_UPDATE_PLAIN + (events / steps + in_ev.numel() / (2 * steps) * (nnz_in / n_in)) * B_PER_EVENT)
                                 * steps / t_f / 1e9 / HBM_PEAK_GBS,
                             "traffic": profile_traffic("training_step_kernels_52k_batch32.txt", "hbm_bytes_per_forward_step")}}
    # the transposed propagation alone, every row active
    lam = torch.randn(L, 4, ne, device="cuda", generator=g)
    gz = torch.empty(8, ne, device="cuda")
    alg = nnz * 8 + ring_bytes + ne * 4
    reps = 50

    def gather_entry(kernel, what, call, traffic_key, traffic_note):
        for k in range(5):
            call(k)
        _, dev = time_region(torch, lambda: [call(k) for k in range(reps)])
        per = dev / reps
        return {"kernel": kernel, "workload": "transposed propagation N=51978 nnz=%d batch=32, every row, %s" % (nnz, what),
                "us_per_launch": per * 1e6, "synapse_trials_per_s": nnz * batch / per,
                "roofline": {"bound": "hbm", "achieved": alg / per / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                             "frac": alg / per / 1e9 / HBM_PEAK_GBS,
                             "what": "HBM-compulsory bytes: table + adjoint ring + output once",
                             "algorithmic_bytes_per_launch": alg,
                             "traffic": profile_traffic("training_step_kernels_52k_batch32.txt", traffic_key),
                             "traffic_note": traffic_note}}

    entries = [step_entry]
    if bptt.blk is not None:
        entries.append(gather_entry(
            "bwd_gather_blocked_kernel", "table regrouped into %d target ranges" % bptt.n_blocks,
            lambda k: ops.csr_propagate_bwd_blocked(bptt.blk, bptt.n_blocks, lam, n, batch, k, gz_parts=gz),
            "hbm_bytes_per_launch_bwd_gather_blocked",
            "HBM bytes; the kernel reads one 128-byte adjoint row per synapse (6.6 GB per launch) from the L2s, "
            "which is what bounds it"))
    entries.append(gather_entry(
        "bwd_gather4_kernel", "source-major table row by row",
        lambda k: ops.csr_propagate_bwd(sim.rec, lam, n, batch, k, gz=gz[0]),
        "l2_fill_bytes_per_launch_bwd_gather4",
        "L2 fills (one 128-byte adjoint row per synapse, served mostly by the memory-side cache), not HBM bytes"))
    return entries


def bench_batched_v1(torch, batch=8, steps=300):
    """The V1-scale network as a batched run, 230,924 neurons x 8 trials, from the settled state, through the
    launch-per-step driver in the form the simulator picks by itself at this batch and rate (spikes pushed into the
    ring as events: 0.02 events per synapse and step) and through the fused pull form (248 k sources, so one bit of
    its activity map stands for several).  Algorithmic bytes: 18 B per synaptic event + 103 B per element update."""
    import numpy as np
    from bmtk_amd import ops, synthetic, training
    from bmtk_amd.simulator import Glif3Simulator
    rng = np.random.default_rng(3)
    par = synthetic.random_cells(rng, N_CLASSES)
    class_id = rng.integers(0, N_CLASSES, N_V1).astype(np.int32)
    _, by_src, _ = synthetic.device_network(N_V1, MEAN_IN, "lognormal", seed=3)
    inp = synthetic.device_input_table(N_IN, N_V1, N_IN_SYN, seed=4, w_scale=IN_W_SCALE)
    in_ptr, in_ev = ops.poisson_events(N_IN, IN_RATE_HZ, 1.0, 600 + 2 * steps, batch=batch, seed=5)
    out = []
    for form, kw in (("the simulator's choice", dict()), ("fused pull form", dict(fused=True))):
        sim = Glif3Simulator(N_V1, par, 1.0, batch=batch, class_id=class_id, rec=by_src, inp=inp, resident=False, **kw)
        sim.set_input_events(in_ptr, in_ev)
        sim.run(600, spike_bits=False)
        sim.run(steps // 4, spike_bits=False)
        res = {}
        wall, dev = time_region(torch, lambda: res.update(out=sim.run(steps)))
        spikes = int(training.spike_counts(res["out"]["bits"], sim.ne).sum().item())
        rec_ev, inp_ev = count_events(torch, sim, res["out"]["bits"], 600 + steps // 4)
        per = dev / steps
        alg = (rec_ev + inp_ev) / steps * B_PER_EVENT + sim.ne * B_PER_UPDATE_CLASS
        out.append({"kernel": "sim_fused_kernel" if sim.fuse_table is not None else "sim_step_kernel",
                    "workload": "V1-scale batched run: 230,924 neurons x %d trials, %d steps, %s" % (batch, steps, form),
                    "activity_map_sources_per_bit": 1 << sim.fuse_shift if sim.fuse_table is not None else None,
                    "us_per_sim_step": per * 1e6, "neuron_updates_per_s": sim.ne / per,
                    "synaptic_events_per_s": (rec_ev + inp_ev) / dev, "mean_rate_hz": spikes / (sim.ne * steps * 1e-3),
                    "roofline": {"bound": "hbm", "achieved": alg / per / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                 "frac": alg / per / 1e9 / HBM_PEAK_GBS, "traffic": None,
                                 "what": "18 B per synaptic event + 103 B per element update"}})
        del sim
    return out


def bench_lds(torch, clock_ghz=2.4):
    """What the LDS and the path between workgroups cost (the figures the resident kernels' design quotes):
    additions into a 92 KB LDS array in five forms with 64, 8 and 1 active lanes per wavefront, in clocks per
    wavefront instruction on a compute unit at a nominal 2.4 GHz, and the time a word takes from one workgroup to
    another through device memory, on one XCD and across two; and the rate of scattered fp32 atomic additions into
    device memory, anywhere and with every XCD confined to an eighth of the region."""
    from bmtk_amd import _lib
    from bmtk_amd.ops import _p, _stream
    lib = _lib.load()
    n_blocks, rounds = 256, 2000
    out_buf = torch.empty(n_blocks * 1024, device="cuda")
    names = {0: "ds_add_f32", 1: "ds_add_u32", 2: "ds_add_u64", 3: "float add by compare-and-swap loop", 4: "plain store"}
    entries = []
    for op in range(5):
        row = {}
        for active in (64, 8, 1):
            call = lambda: _lib.check(lib.bmtk_microbench_lds(op, active, rounds, n_blocks, _p(out_buf), _stream()))
            call()
            _, dev = time_region(torch, lambda: [call() for _ in range(5)])
            clk = dev / 5 * clock_ghz * 1e9 / (16.0 * rounds)     # 16 wavefronts per compute unit, one workgroup each
            row[str(active) + " lanes"] = {"clocks_per_wavefront_instruction": clk, "clocks_per_lane": clk / active}
        entries.append({"kernel": "lds_add_kernel", "workload": "LDS addition, " + names[op], "result": row,
                        "clock_ghz_assumed": clock_ghz})
    flags = torch.zeros(1024, dtype=torch.int32, device="cuda")
    xcc = torch.zeros(4, dtype=torch.int32, device="cuda")
    hop_rounds = 20000
    for a, b, what in ((0, 8, "workgroups 0 and 8"), (0, 1, "workgroups 0 and 1")):
        best = None
        for _ in range(3):
            flags.zero_(); xcc.zero_()
            _, dev = time_region(torch, lambda: _lib.check(lib.bmtk_microbench_hop(_p(flags), _p(xcc), a, b, hop_rounds,
                                                                                   1_000_000, _stream())))
            best = dev if best is None else min(best, dev)
        x = xcc.cpu().tolist()
        entries.append({"kernel": "hop_kernel", "workload": "word passed between two workgroups through device memory, " + what,
                        "xcd_of_each": x[:2], "gave_up": bool(x[2]), "us_per_hop": best / hop_rounds / 2 * 1e6})
    # scattered fp32 atomic additions into device memory: what holds the event-driven propagation forms
    per_thread, blocks = 64, 8192
    for mb in (4, 53, 400):
        cells = torch.zeros(mb * (1 << 20) // 32 * 8, device="cuda")
        for own in (0, 1):
            best = None
            for _ in range(3):
                cells.zero_()
                _, dev = time_region(torch, lambda: _lib.check(lib.bmtk_microbench_atomics(
                    _p(cells), cells.numel(), per_thread, blocks, own, _stream())))
                best = dev if best is None else min(best, dev)
            total = blocks * 256 * per_thread
            entries.append({"kernel": "atomic_add_kernel",
                            "workload": "fp32 atomic additions to random cells of %d MB, %s" % (
                                mb, "each workgroup within its XCD's eighth" if own else "anywhere"),
                            "atomics_per_s": total / best, "none_lost": float(cells.double().sum().item()) == float(total)})
        del cells
    return entries


def bench_small_network(torch):
    """The size of the reference's own examples: configuration 0's 450 neurons, which ONE workgroup holds (the
    single-workgroup form of the resident kernel), with the spike record on as the front ends run it."""
    from bmtk_amd import synthetic
    from bmtk_amd.simulator import Glif3Simulator
    out = []
    cfg = synthetic.small_glif3_network(n=450, n_in=1000, steps=21000, seed=0, in_w_scale=2.0)
    small = Glif3Simulator(cfg["n"], cfg["par"], cfg["h"], rec=cfg["rec_src"], inp=cfg["inp_src"], ring_slots=cfg["L"])
    small.set_input_events(cfg["in_ptr"], cfg["in_events"])
    small.run(1000)
    wall, dev = time_region(torch, lambda: small.run(20000, spike_bits=False, record_cap=1 << 20))
    small.check()
    out.append({"kernel": "sim_solo_kernel (one workgroup, spike record on)",
                "workload": "450 GLIF3 neurons (configuration 0's network), 20000 steps", "groups": small.res_groups,
                "us_per_sim_step": dev / 20000 * 1e6, "neuron_updates_per_s": 450 * 20000 / wall,
                "roofline": {"bound": "hbm", "achieved": 450 * B_PER_UPDATE_PLAIN * 20000 / dev / 1e9, "peak": HBM_PEAK_GBS,
                             "unit": "GB/s", "frac": 450 * B_PER_UPDATE_PLAIN * 20000 / dev / 1e9 / HBM_PEAK_GBS,
                             "traffic": None, "what": "one workgroup on one compute unit: bound by instruction issue (about 2,200 instructions per step over its 16 wavefronts), not by memory"}})
    return out


def bench_front_end(torch, sim, steps):
    """What a run through the front ends costs (bmtk_amd.nest.Simulate, bmtk_amd.pointnet.PointSimulator.run): the same
    V1-scale simulation with the spike record on (spike times need the crossing fraction), then the record joined,
    ordered by spike time on the device and copied to the host.  And the size of the reference's own examples: 450
    neurons, which one workgroup holds."""
    import numpy as np
    from bmtk_amd import synthetic
    from bmtk_amd.simulator import Glif3Simulator
    res = {}

    def run():
        res["out"] = sim.run(steps, spike_bits=False, record_cap=steps * N_V1 // 8)

    run()
    wall, dev = time_region(torch, run)
    t0 = time.perf_counter()
    rec = sim.collect_record(res["out"]["record"], sort_scale=1.0)
    times, senders = sim.to_host(rec["time"], rec["elem"])
    collect = time.perf_counter() - t0
    alg_step = N_V1 * B_PER_UPDATE_CLASS   # the state update alone; the events ride on top as in the headline
    out = [{"kernel": "sim_resident_kernel (spike record on) + collect_record",
            "workload": "V1-scale forward simulation as the front ends run it, %d steps" % steps,
            "us_per_sim_step": dev / steps * 1e6, "neuron_updates_per_s": N_V1 * steps / wall,
            "spikes": int(times.size), "record_overflow": bool(rec["overflow"]),
            "collect_sort_copy_ms": collect * 1e3,
            "roofline": {"bound": "hbm", "achieved": alg_step * steps / dev / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": alg_step * steps / dev / 1e9 / HBM_PEAK_GBS, "traffic": None,
                         "what": "state update bytes only (103 B per neuron and step)"}}]
    out += bench_small_network(torch)
    return out


def cpu_baseline(torch, sim, par, class_id, settled, sample_steps):
    """The NEST-algorithm CPU restatement (fp64, event-driven source-major delivery into per-neuron ring
    buffers, OpenMP) on `sample_steps` steps of the same network, started from the settled state the GPU's
    timed region started from (copied to the host), so that it sees the same activity."""
    import numpy as np
    from oracle import glif3_oracle as orc
    rec = tuple(t.cpu().numpy() for t in (sim.rec.indptr, sim.rec.indices, sim.rec.weights, sim.rec.delays,
                                          sim.rec.receptors))
    inp = tuple(t.cpu().numpy() for t in (sim.inp.indptr, sim.inp.indices, sim.inp.weights, sim.inp.delays,
                                          sim.inp.receptors))
    in_ptr = sim.in_ptr.cpu().numpy()
    in_ev = sim.in_events.cpu().numpy()
    prop = orc.precompute(par, 1.0)
    step0 = settled["step"]
    res = {}
    for label, threads, steps in (("all", orc.max_threads(), sample_steps), ("one", 1, max(CPU_MIN_STEPS, sample_steps // 10))):
        orc.set_threads(threads)
        st = {k: np.ascontiguousarray(v, np.int32 if k == "ref" else np.float64) for k, v in settled["state"].items()}
        ring = np.ascontiguousarray(settled["ring"], np.float64)
        t0 = time.perf_counter()
        out = orc.simulate(st, prop, 1.0, steps, class_id=class_id, ring=ring, rec=rec, inp=inp, in_ptr=in_ptr,
                           in_events=in_ev, spike_cap=max(1024, steps * N_V1 // 16), step0=step0)
        dt = time.perf_counter() - t0
        deg = np.diff(rec[0])
        ev = int(deg[out["elem"]].sum()) + int(np.diff(inp[0])[in_ev[in_ptr[step0]:in_ptr[step0 + steps]]].sum())
        res[label] = dict(threads=threads, steps=steps, seconds=dt, updates_per_s=N_V1 * steps / dt,
                          events_per_s=ev / dt, rate_hz=out["count"] / (N_V1 * steps * 1e-3))
    orc.set_threads(res["all"]["threads"])
    a, o = res["all"], res["one"]
    return {"value": a["updates_per_s"], "unit": "neuron-updates/s", "cores": a["threads"], "kind": "port",
            "sample": "%d steps of the same 230,924-neuron network from the settled state the GPU run was timed "
                      "from (%.1f s, %.2f Hz mean rate); NEST-algorithm restatement in C, fp64, OpenMP, not NEST"
                      % (a["steps"], a["seconds"], a["rate_hz"]),
            "synaptic_events_per_s": a["events_per_s"],
            "one_thread": {"value": o["updates_per_s"], "synaptic_events_per_s": o["events_per_s"],
                           "steps": o["steps"], "seconds": o["seconds"]},
            "host_cpu_count": os.cpu_count()}


def settle(torch, sim, min_steps=SETTLE_STEPS, max_steps=SETTLE_MAX_STEPS, block=100):
    """Run the network, untimed, until it has left the transient from rest: at least `min_steps` steps and
    then until the spike count of a block of 100 steps lies within 10 % of the mean of the three blocks before it
    (or `max_steps`).  Returns the number of steps taken."""
    from bmtk_amd import training
    counts, done = [], 0
    while done < max_steps:
        out = sim.run(block)
        counts.append(int(training.spike_counts(out["bits"], sim.ne).sum().item()))
        done += block
        if done >= min_steps and len(counts) >= 4:
            prev = sum(counts[-4:-1]) / 3.0
            if prev > 0 and abs(counts[-1] - prev) <= 0.1 * prev:
                break
    sim.check()
    return done, counts


def unscaled_activity(torch, steps=200, settle_steps=400):
    """The same network with the input weights as specified (lognormal(0,1) x 1 pA, not x 7): mean rate and synaptic
    events per step over `steps` steps after `settle_steps` from rest, untimed -- what the x 7 of the timed network
    is a deviation from."""
    from bmtk_amd import training
    sim, _, _ = build_v1(torch, settle_steps + steps, in_w_scale=1.0)
    sim.run(settle_steps, spike_bits=False)
    out = sim.run(steps)
    sim.check()
    rec, inp = count_events(torch, sim, out["bits"], settle_steps)
    spikes = int(training.spike_counts(out["bits"], sim.ne).sum().item())
    return {"input_weight_scale": 1.0, "steps": steps, "settle_steps": settle_steps, "spikes": spikes,
            "mean_rate_hz": spikes / (N_V1 * steps * 1e-3), "recurrent_events_per_sim_step": rec / steps,
            "input_events_per_sim_step": inp / steps, "events_per_sim_step": (rec + inp) / steps}


def launch_overhead(torch, sim, n1=100, n2=1100, reps=3):
    """Fixed cost of one `bmtk_glif3_simulate_fwd` call as the intercept of two run lengths (HIP events, best
    of `reps`): (seconds per step at the margin, fixed seconds per call)."""
    best = {}
    for n in (n1, n2):
        ts = []
        for _ in range(reps):
            _, dev = time_region(torch, lambda: sim.run(n, spike_bits=False))
            ts.append(dev)
        best[n] = min(ts)
    slope = (best[n2] - best[n1]) / (n2 - n1)
    return slope, best[n1] - slope * n1


def kernel_summary(kernels):
    """{short name: {us, frac, ...}} of the isolated-kernel entries: state update (both forms), propagation (every
    form and rate), the training step."""
    out = {}
    for k in kernels:
        w, r = k["workload"], k.get("roofline", {})
        if w.startswith("state update"):
            name = "state_update_class_table" if "class table" in w else "state_update_per_neuron_parameters"
            out[name] = {"us_per_launch": k["us_per_launch"], "neuron_updates_per_s": k["neuron_updates_per_s"],
                         "frac": r.get("frac"), "traffic": r.get("traffic"),
                         # measured HBM bytes (profile) / this run's launch time / peak
                         "hbm_frac": None if not r.get("traffic") else
                         r["traffic"] / (k["us_per_launch"] * 1e-6) / 1e9 / HBM_PEAK_GBS}
        elif w.startswith("propagation"):
            rate = w.split("rate=")[1]
            out.setdefault("propagation_us_per_arrival_step", {}).setdefault(rate, {})[k["kernel"].split(" ")[0].rstrip(":")] = \
                round(k["us_per_arrival_step"], 1)
            if k["kernel"].startswith(("pull", "auto")):
                out.setdefault("propagation_frac", {}).setdefault(rate, {})[k["kernel"].split(" ")[0].rstrip(":")] = \
                    {"frac": r.get("frac"), "hbm_frac": r.get("hbm_frac"), "events_per_s": k["synaptic_events_per_s"]}
        elif w.startswith("BPTT step"):
            out["bptt_step"] = {"forward_s": k["forward_s"], "backward_s": k["backward_s"],
                                "forward_us_per_step": k["forward_s"] / 600 * 1e6,
                                "backward_frac": r.get("frac"), "forward_frac": k["roofline_forward"]["frac"],
                                "weight_grad_events_per_s": k["weight_grad_events_per_s"]}
        elif w.startswith("V1-scale batched run"):
            out["v1_scale_batch_8, " + ("fused pull form" if "fused" in w else "the simulator's choice")] = {"us_per_sim_step": k["us_per_sim_step"], "neuron_updates_per_s": k["neuron_updates_per_s"],
                                       "synaptic_events_per_s": k["synaptic_events_per_s"], "frac": r.get("frac")}
        elif w.startswith("transposed propagation"):
            out.setdefault("transposed_propagation_us", {})[k["kernel"]] = round(k["us_per_launch"], 1)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5,
                    help="timed passes; one pass = one call of the forward simulation over --sim-steps steps of "
                         "1 ms (what one nest.Simulate(tstop) does for the reference)")
    ap.add_argument("--warmup", type=int, default=1, help="untimed passes before the timed ones")
    ap.add_argument("--sim-steps", type=int, default=SIM_STEPS,
                    help="simulation steps per pass (the configuration's 3000)")
    ap.add_argument("--cpu-steps", type=int, default=3000, help="steps of the CPU baseline sample (0 = skip)")
    ap.add_argument("--no-kernels", action="store_true", help="skip the isolated-kernel measurements")
    ap.add_argument("--kernels", default="state,compaction,propagation,bptt,batched_v1",
                    help="which isolated-kernel measurements to run (comma-separated)")
    ap.add_argument("--propagation-modes", default=",".join(PROPAGATION_MODES),
                    help="delivery forms the propagation group times (profiler runs leave out 'auto', which launches "
                         "the scatter and gather kernels too and would be pooled with them)")
    ap.add_argument("--propagation-rates", default=",".join("%g" % r for r in PROPAGATION_RATES),
                    help="firing rates (Hz) the propagation group times (profiler runs take one at a time, so that a "
                         "kernel's launches are not pooled over the rates)")
    ap.add_argument("--kernels-in-line", action="store_true",
                    help="put the full isolated-kernel entries into the result line (default: a short kernel_summary "
                         "in the line, the full entries as a JSON line on stderr)")
    ap.add_argument("--only-kernels", action="store_true",
                    help="run only the isolated-kernel measurements of --kernels (for profiler runs); prints a line "
                         "with just their entries")
    ap.add_argument("--per-step", action="store_true", help="force one launch per step instead of resident mode")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run a 1 GiB device-to-device copy 10 times (reference for scaling the FETCH_SIZE / "
                         "WRITE_SIZE counters) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (the path is not sharded); use --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    from bmtk_amd import _lib, training
    _lib.load()
    if args.calibrate_copy:
        src = torch.ones(1 << 28, device="cuda")       # 1 GiB of fp32
        dst = torch.empty_like(src)
        for _ in range(10):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibrate_copy_bytes_read": src.numel() * 4, "bytes_written": src.numel() * 4, "copies": 10}))
        return

    modes = tuple(m for m in args.propagation_modes.split(",") if m)
    rates = tuple(float(r) for r in args.propagation_rates.split(",") if r)
    if set(modes) - set(PROPAGATION_MODES):
        sys.exit("bench.py: --propagation-modes takes %s" % ", ".join(PROPAGATION_MODES))
    groups = {"state": bench_state_update, "compaction": bench_compaction,
              "propagation": lambda t: bench_propagation(t, modes=modes, rates=rates), "bptt": bench_bptt,
              "small": bench_small_network, "batched_v1": bench_batched_v1, "lds": bench_lds}   # (the headline run reports "small" with its front-end entries)
    want = [g for g in args.kernels.split(",") if g]
    unknown = set(want) - set(groups)
    if unknown:
        sys.exit("bench.py: unknown --kernels entries: %s" % ", ".join(sorted(unknown)))
    if args.only_kernels:
        print(json.dumps({"only_kernels": True, "kernels": sum((groups[g](torch) for g in groups if g in want), [])}))
        return

    K, W, S = args.steps, args.warmup, args.sim_steps
    if K < 1 or W < 0 or S < 1:
        sys.exit("bench.py: --steps and --sim-steps must be positive, --warmup non-negative")
    if K * S * ((N_V1 + 63) // 64) * 8 > 100e9:
        sys.exit("bench.py: --steps x --sim-steps spike bits would exceed 100 GB; use fewer passes")
    overhead_steps = 3 * (100 + 1100) + 2 * S      # launch-overhead runs and the front-end entry
    sim, par, class_id = build_v1(torch, SETTLE_MAX_STEPS + (W + K) * S + overhead_steps,
                                  resident=False if args.per_step else "auto")
    # untimed: leave the transient from rest behind, whatever --warmup says
    settled_steps, settle_counts = settle(torch, sim)
    torch.cuda.synchronize()
    settled = {"step": sim.step, "state": sim.state.to_numpy(), "ring": sim.ring.cpu().numpy()}
    for _ in range(W):
        sim.run(S, spike_bits=False)
    step_timed = sim.step
    passes = []
    wall, dev = time_region(torch, lambda: [passes.append(sim.run(S)) for _ in range(K)])
    sim.check()
    rec_ev = in_ev = n_spikes = 0
    for k, out in enumerate(passes):
        r, i = count_events(torch, sim, out["bits"], step_timed + k * S)
        rec_ev, in_ev = rec_ev + r, in_ev + i
        n_spikes += int(training.spike_counts(out["bits"], sim.ne).sum().item())
        out["bits"] = None
    events = rec_ev + in_ev
    total_steps = K * S
    resident = bool(sim.res_span)
    # resident mode: every pass is ONE launch of sim_resident_kernel covering its S steps;
    # otherwise S+1 launches of sim_step_kernel per pass
    launches = K if resident else K * (S + 1)
    per_launch = dev / launches
    alg_step = N_V1 * B_PER_UPDATE_CLASS + events / total_steps * B_PER_EVENT
    alg = alg_step * total_steps / launches
    slope, fixed = launch_overhead(torch, sim)
    sim.check()
    traffic_step = profile_traffic("sim_resident_kernel_v1_forward_230k.txt" if resident else
                                   "sim_step_kernel_v1_forward_230k_per_step_launches.txt", "hbm_bytes_per_step")
    line = {
        "metric": "neuron-updates/s (with synaptic events/s) at 230k neurons; % of HBM roofline",
        "value": N_V1 * total_steps / wall, "unit": "neuron-updates/s",
        "synaptic_events_per_s": events / wall,
        "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": wall / K * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "V1-scale forward simulation: 230,924 GLIF3 neurons, 111 classes, %d recurrent + %d "
                               "input synapses, 17,400 Poisson inputs at 5 Hz, dt 1 ms, batch 1, %d simulation steps "
                               "per pass" % (sim.rec.nnz, sim.inp.nnz, S),
                   "step_definition": "one pass = one forward-simulation call over %d steps of 1 ms (one "
                                      "nest.Simulate(tstop) of the reference); --steps counts passes" % S,
                   "sim_steps_per_pass": S, "sim_steps_timed": total_steps,
                   "settle_steps_untimed": settled_steps, "settle_spikes_per_100_steps": settle_counts[-4:],
                   "mode": "resident (one cooperative launch per pass)" if resident else "one launch per step",
                   "mean_rate_hz": n_spikes / (N_V1 * total_steps * 1e-3),
                   "spikes": n_spikes, "recurrent_events": rec_ev, "input_events": in_ev,
                   "events_per_sim_step": events / total_steps, "us_per_sim_step": wall / total_steps * 1e6,
                   "input_weight_scale": IN_W_SCALE,
                   "same_network_at_input_weight_x1": unscaled_activity(torch)},
        "roofline": {"bound": "hbm", "kernel": "sim_resident_kernel" if resident else "sim_step_kernel",
                     "achieved": alg / per_launch / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": alg / per_launch / 1e9 / HBM_PEAK_GBS,
                     "traffic": None if traffic_step is None else traffic_step * total_steps / launches,
                     "traffic_source": "profiles/ (rocprofv3 FETCH_SIZE + WRITE_SIZE summary; a constant of that "
                                       "profile run, not re-measured here)",
                     "launches": launches, "algorithmic_bytes_per_launch": alg, "us_per_launch": per_launch * 1e6,
                     "algorithmic_bytes_per_step": alg_step, "us_per_step": dev / total_steps * 1e6,
                     "launch_overhead_us": fixed * 1e6, "marginal_us_per_step": slope * 1e6,
                     "frac_at_the_margin": alg_step / slope / 1e9 / HBM_PEAK_GBS},
    }
    kernels = None
    if not args.no_kernels:
        del passes
        kernels = (bench_front_end(torch, sim, S) if resident else []) + \
            sum((groups[g](torch) for g in groups if g in want), [])
        # the figures the other kernels are judged by, once more and short, ahead of the long list
        line["kernel_summary"] = kernel_summary(kernels)
    if args.cpu_steps > 0:
        line["cpu_baseline"] = cpu_baseline(torch, sim, par, class_id, settled, max(CPU_MIN_STEPS, args.cpu_steps))
    if kernels is not None:
        # The full entries are long (every form and rate): they go to stderr as a JSON line of their own unless asked
        # for in the result line, which stays short enough to be kept whole by whatever records it.
        if args.kernels_in_line:
            line["kernels"] = kernels
        else:
            print(json.dumps({"kernels": kernels}), file=sys.stderr, flush=True)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
