"""Headline benchmark: network evaluations per second at batch 4096, int8, one MI355X.

One step = one launch of the evaluator over one batch of synthetic positions (seeded
random playouts of 0-120 plies, with legal-move masks ANDed in-kernel); inputs are resident
in HBM and outputs preallocated before the timed region.  Prints ONE JSON line.

Extra objects in the line:
  roofline      dense-int8 MFMA roofline of the evaluator kernel: algorithmic int8 ops per
                launch (402,653,184 per evaluation x batch) over the kernel's average duration
                measured with HIP events on the launch stream; `measured_mfma_rate` is the rate
                a register-resident loop of the same MFMA instruction reaches on this GPU (TOP/s).
  cpu_baseline  the CPU port of the same forward (oracle/emulated.py, PyTorch on the host
                cores) timed on a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

OPS_PER_EVAL = 402_653_184            # 2 * 32 tokens * 8 layers * 12 * 256^2 int8 ops in the weight GEMMs
OPS_PER_EVAL_STRESS = 3_221_225_472   # 2 * 32 tokens * 16 layers * 12 * 512^2 (the 512-wide, 16-layer network)
PEAK_INT8_OPS = 5.0e15                # MI355X dense int8 MFMA, ops/s
PEAK_FP16_OPS = 2.5e15                # dense fp16 MFMA: the e4m3 format's products run on the fp16 instruction
# HBM bytes per launch from the FETCH_SIZE / WRITE_SIZE counter runs summarised under profiles/
# (calibrated on a 1 GiB copy), by (network shape, kernel, batch).
MEASURED_TRAFFIC_BYTES = {("base", "duo", 4096): 0.445e9, ("base", "twin", 4096): 0.78e9, ("base", "quad", 4096): 3.07e9,
                          ("base", "board", 256): 5.5e7, ("base", "octo", 256): 5.5e7, ("stress", "board", 16384): 2.66e10,
                          ("stress", "octo", 16384): 2.95e10}
MEASURED_TRAFFIC_BYTES_E4M3 = {("base", "twin", 4096): 0.97e9}
# vector-ALU instructions per launch (SQ_INSTS_VALU of the same counter runs), by (network shape, kernel, batch):
# with the matrix products hidden, the launch cannot be shorter than these instructions' issue time
MEASURED_VALU_INSTS = {("base", "duo", 4096): 5.938e8, ("base", "twin", 4096): 5.513e8}
SIMDS, CLOCK_HZ = 1024, 2.4e9
PEAK_HBM_BPS = 8.0e12                 # MI355X HBM3E, bytes/s


def cpu_baseline(net, batch: int, threads: int, budget_s: float = 20.0, mode: str = "int8", plies: int = 80):
    """The int8- (or e4m3-) simulated forward of oracle/emulated.py on the host cores (a port,
    not the reference's files, which do not travel)."""
    import torch
    from brokefish_amd import positions
    from oracle import emulated
    sd = {k: v.detach() for k, v in net.state_dict().items()}
    b, c, r, m = positions.random_positions(batch, plies=plies, seed=0)   # configs[0]: playouts of 0-80 plies
    torch.set_num_threads(threads)
    with torch.no_grad():
        t0 = time.perf_counter()
        emulated.forward(sd, b, c, r, mode=mode, mask=m)               # warm-up, also sizes the loop
        one = time.perf_counter() - t0
        reps = max(2, min(20, int(budget_s / max(one, 1e-3))))
        times = []
        for _ in range(reps):
            t0 = time.perf_counter()
            emulated.forward(sd, b, c, r, mode=mode, mask=m)
            times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {"value": batch / med, "unit": "evals/s", "cores": threads, "kind": "port",
            "sample": f"{reps} reps of batch {batch}, seeded random playouts of 0-{plies} plies ({mode}-simulated PyTorch forward, median), "
                      f"os.cpu_count()={os.cpu_count()}"}


def physical_cores() -> int:
    """Physical cores this process may run on: distinct (package, core) pairs of /proc/cpuinfo among the
    CPUs of the affinity mask (hardware threads of one core count once)."""
    try:
        allowed = os.sched_getaffinity(0)
        seen, cpu, phys = set(), None, 0
        for line in open("/proc/cpuinfo"):
            k, _, v = line.partition(":")
            k, v = k.strip(), v.strip()
            if k == "processor":
                cpu = int(v)
            elif k == "physical id":
                phys = int(v)
            elif k == "core id" and cpu in allowed:
                seen.add((phys, int(v)))
        return len(seen) or len(allowed)
    except OSError:
        return os.cpu_count() or 1


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=None, help="default 4096 (base) / 16384 (stress)")
    ap.add_argument("--quant", choices=("int8", "e4m3"), default="int8",
                    help="operand format of the weight matmuls; int8 is the headline metric, e4m3 the fp8 variant")
    ap.add_argument("--shape", choices=("base", "stress"), default="base",
                    help="base: 8 layers, width 256 (the headline metric); stress: 16 layers, width 512, "
                         "16 heads, default batch 16384")
    ap.add_argument("--kernel", choices=("auto", "quad", "board", "twin", "octo", "duo"), default="auto",
                    help="four positions per workgroup (quad); one position per workgroup with one (board; octo: eight wavefronts) or two (twin) workgroups per compute unit; two positions per workgroup (duo); auto: by batch size and format")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-batch", type=int, default=64)
    ap.add_argument("--no-extras", action="store_true",
                    help="headline only: skip the batch sweep, the e4m3 and stress configurations and the parity report")
    ap.add_argument("--sweep", action="store_true", help="(kept for older command lines: the sweep is part of the default line)")
    ap.add_argument("--copy-probe-mib", type=int, default=0,
                    help="also run one device copy of this many MiB (a kernel of known HBM traffic, "
                         "to calibrate FETCH_SIZE / WRITE_SIZE counter runs)")
    ap.add_argument("--phases", action="store_true",
                    help="add `phases` to the line: shader-clock ticks per wavefront and phase from the profiling "
                         "build of the selected kernel")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this path runs on one GPU (positions shard with no exchange step); --gpus must be 1",
              file=sys.stderr)
        return 2

    import torch
    from brokefish_amd import encoder_impl, positions
    from brokefish_amd.net import BrokefishNet

    stress = a.shape == "stress"
    headline = not stress and a.quant == "int8" and a.batch in (None, 4096)
    if a.batch is None:
        a.batch = 16384 if stress else 4096
    ops_per_eval = OPS_PER_EVAL_STRESS if stress else OPS_PER_EVAL
    torch.manual_seed(0)
    # seed-0 random init, reference init rules
    net = (BrokefishNet(d_model=512, n_heads=16, d_ff=2048, n_layers=16) if stress else BrokefishNet()).eval()
    fp8 = a.quant == "e4m3"
    # fp16 logits: the search contract
    model = encoder_impl("hip")(net, fp8=True, kernel=a.kernel) if fp8 else encoder_impl("hip")(net, int8=True, kernel=a.kernel)
    b, c, r, m = positions.random_positions(a.batch, plies=120, seed=0)
    bd, cd, rd, md = b.cuda(), c.cuda(), r.cuda(), m.cuda()

    if a.copy_probe_mib:
        src = torch.empty(a.copy_probe_mib << 20, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    # The kernel's own duration (HIP events around back-to-back launches on the launch stream) and
    # the two measured ceilings come first: a GPU that has just been woken runs its first tens of
    # milliseconds below its steady clocks, and the timed steps below are meant to see the device as
    # a running search or serving loop sees it.  Short launches are timed over enough repetitions
    # for the clocks to settle.
    from brokefish_amd.hip_impl import mfma_rate, stream_rate
    kname = model.kernel_choice(a.batch)
    kern_ms = model.time_kernel_ms(bd, cd, rd, md, warmup=10 if a.batch <= 1024 else 3 if stress else 40,
                                   iters=max(a.steps, 200 if a.batch <= 1024 else 10))
    stream_ceiling = stream_rate(6_389_760 if kname == "quad" else 50_626_560 if stress else 6_455_296, workgroups=min(a.batch, 4096),
                                 reps=1 if stress else 3)
    measured_mfma = mfma_rate(a.quant)

    # the contract's measurement: W untimed steps, then exactly K steps between two synchronisations
    for _ in range(a.warmup):
        model.forward_full(bd, cd, rd, md)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        model.forward_full(bd, cd, rd, md)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_step = dt / a.steps * 1e3
    evals = a.batch * a.steps / dt
    achieved = ops_per_eval * a.batch / (kern_ms * 1e-3) / 1e12
    peak = PEAK_FP16_OPS if fp8 else PEAK_INT8_OPS
    traffic = (MEASURED_TRAFFIC_BYTES_E4M3 if fp8 else MEASURED_TRAFFIC_BYTES).get((a.shape, kname, a.batch))
    # each workgroup streams its own copy of the weights from L2
    # (four positions share one copy in the quad kernel, two in the duo kernel)
    weight_bytes = (6_389_760 * ((a.batch + 3) // 4) if kname == "quad" else 6_455_296 * ((a.batch + 1) // 2) if kname == "duo"
                    else (50_626_560 if stress else 6_455_296) * a.batch)
    line = {
        "metric": (f"network evals/sec at batch {a.batch} int8, 16-layer width-512 stress shape, on 1 MI355X" if stress
                   else f"network evals/sec at batch 4096 {'fp8 e4m3' if fp8 else 'int8'} on 1 MI355X"),
        "value": evals, "unit": "evals/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8" if fp8 else "int8", "data": "synthetic",
        "config": {"workload": (f"configs[4]: 16-layer d512 16-head FFN2048 int8 evaluator, batch {a.batch}, " if stress else
                                f"configs[{3 if fp8 else 1}]: 8-layer d256 8-head FFN1024 {a.quant} evaluator, batch {a.batch}, ")
                               + f"kernel {kname}, binding {model.binding}, "
                               "seeded random playouts 0-120 plies, legal-move mask ANDed in-kernel, "
                               "fp16 logits out, seed-0 random-init weights"},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": peak / 1e12, "unit": "TFLOP/s" if fp8 else "TOP/s",
                     "frac": achieved / (peak / 1e12),
                     # HBM bytes per launch: not measurable inside this process; the figure is the
                     # FETCH_SIZE + WRITE_SIZE counter result of the same command summarised under profiles/
                     "traffic": traffic, "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summaries under profiles/ (not measured in this run)" if traffic else None,
                     "kernel_ms": kern_ms, "ops_per_launch": ops_per_eval * a.batch,
                     # what the launch cannot go below with every matrix product hidden: the vector instructions
                     # the bit-exact fp32 / fp64 epilogues, LayerNorm, softmax and quantisers take, at four clocks
                     # each on 1024 SIMDs (instruction count from the counter runs under profiles/, like `traffic`)
                     "valu_floor_ms": (MEASURED_VALU_INSTS[(a.shape, kname, a.batch)] * 4 / (SIMDS * CLOCK_HZ) * 1e3
                                       if not fp8 and (a.shape, kname, a.batch) in MEASURED_VALU_INSTS else None),
                     "limiter": "vector ALU + fp32 matrix instructions (softmax, epilogues, quantisers); the int8 products are hidden under them",
                     # the kernel's second resource: every position streams the packed weights out of the
                     # cache hierarchy (bytes_per_launch / kernel_ms = achieved); `stream_ceiling_TBps` is
                     # what the same number of workgroups reach streaming a buffer of the network's size
                     # with nothing else to do (measured below), `l1_fill_nominal_TBps` 64 bytes per clock
                     # and compute unit
                     "weight_stream": {"bytes_per_launch": weight_bytes, "achieved_TBps": weight_bytes / (kern_ms * 1e-3) / 1e12,
                                       "l1_fill_nominal_TBps": 256 * 64 * 2.4e9 / 1e12}},
    }
    line["roofline"]["weight_stream"]["stream_ceiling_TBps"] = stream_ceiling
    # the matrix pipe's measured ceiling for the instruction the kernel uses (register-resident
    # MFMA chains, no memory traffic), next to the datasheet peak that `frac` is quoted against
    line["roofline"]["measured_mfma_rate"] = measured_mfma
    line["step_protocol"] = (f"{a.warmup} untimed steps, then {a.steps} steps between two device synchronisations; "
                             "the kernel timing and the ceiling probes ran before them (device at its steady clocks)")
    if a.phases:
        ph = model.profile_phases(bd, cd, rd, md)
        line["phases"] = {"kernel": kname, "ticks_per_wavefront": {k: round(v, 1) for k, v in ph.items()},
                          "share_of_total": {k: round(v / ph["total"], 4) for k, v in ph.items() if k != "total"}}
    del model, bd, cd, rd, md
    if headline and not a.no_extras:
        # configurations 3, 4 and 5 timed in interleaved rounds (every point once per round, median over the
        # rounds), as the reference's bench does for its variants (bench/bench_model.py:167-193): the batch
        # sweep (small-batch latency regime; same net, same generator), e4m3 at batch 4096 (products on the
        # fp16 matrix instruction: quoted against both peaks), the 16-layer 512-wide network at batch 16384
        torch.manual_seed(0)
        wide = BrokefishNet(d_model=512, n_heads=16, d_ff=2048, n_layers=16).eval()
        hip = encoder_impl("hip")
        mdl8, mdlf, mdlw = hip(net, int8=True, kernel=a.kernel), hip(net, fp8=True, kernel=a.kernel), hip(wide, int8=True)
        points = [("sweep", nb, mdl8, 200 if nb <= 256 else 60 if nb <= 1024 else 20 if nb <= 16384 else 6) for nb in (64, 256, 1024, 4096, 16384, 65536)]
        points += [("e4m3", 4096, mdlf, 20), ("stress", 16384, mdlw, 4)]
        inputs = {nb: [t.cuda() for t in positions.random_positions(nb, plies=120, seed=0)] for nb in {p[1] for p in points}}
        rounds = 3
        times = {(p[0], p[1]): [] for p in points}
        for _ in range(rounds):
            for name, nb, mdl, iters in points:
                times[(name, nb)].append(mdl.time_kernel_ms(*inputs[nb], warmup=2, iters=iters))
        med = {k: sorted(v)[len(v) // 2] for k, v in times.items()}
        line["sweep"] = [{"batch": nb, "ms_per_launch": med[("sweep", nb)], "evals_per_s": nb / med[("sweep", nb)] * 1e3,
                          "kernel": mdl8.kernel_choice(nb), "frac_int8_peak": OPS_PER_EVAL * nb / (med[("sweep", nb)] * 1e-3) / PEAK_INT8_OPS,
                          "ms_min_max": [min(times[("sweep", nb)]), max(times[("sweep", nb)])]}
                         for nb in (64, 256, 1024, 4096, 16384, 65536)]
        line["timing_protocol"] = f"{rounds} interleaved rounds over the sweep, e4m3 and stress points, median; HIP events on the launch stream"
        ms = med[("e4m3", 4096)]
        tops = OPS_PER_EVAL * 4096 / (ms * 1e-3)
        line["e4m3"] = {"batch": 4096, "kernel": mdlf.kernel_choice(4096), "kernel_ms": ms, "evals_per_s": 4096 / ms * 1e3, "achieved_TFLOPs": tops / 1e12,
                        "frac_fp16_peak_2.5PF": tops / PEAK_FP16_OPS, "frac_fp8_peak_5.0PF": tops / 5.0e15,
                        "measured_mfma_rate": mfma_rate("e4m3")}
        ms = med[("stress", 16384)]
        line["stress"] = {"batch": 16384, "kernel": mdlw.kernel_choice(16384), "kernel_ms": ms, "evals_per_s": 16384 / ms * 1e3,
                          "achieved_TOPs": OPS_PER_EVAL_STRESS * 16384 / (ms * 1e-3) / 1e12,
                          "frac_int8_peak": OPS_PER_EVAL_STRESS * 16384 / (ms * 1e-3) / PEAK_INT8_OPS}
        line["neighbours"] = neighbours(mdl8, inputs)
        del mdl8, mdlf, mdlw, wide, inputs
        line["parity"] = parity_report(net)
    if not a.no_cpu:
        cores = physical_cores()
        threads = max(1, min(cores, int(os.environ.get("OMP_NUM_THREADS", "16"))))
        line["cpu_baseline"] = cpu_baseline(net, a.cpu_batch, threads, mode=a.quant, budget_s=12.0)
        line["cpu_baseline"]["physical_cores"] = cores
        if headline and not a.no_extras:      # configuration 1 names fp32 and the int8 simulation
            f32 = cpu_baseline(net, a.cpu_batch, threads, mode="fp32", budget_s=4.0)
            line["cpu_baseline"]["fp32"] = {"value": f32["value"], "unit": "evals/s", "sample": f32["sample"]}
    print(json.dumps(line))
    return 0


def neighbours(model, inputs):
    """The kernels either side of the evaluator -- legal-move generation in front, the search's edge
    expansion behind -- timed alone with events on the launch stream, with their algorithmic bytes
    against the HBM peak (integer / byte work: 67 B of position in and 257 B of mask and check flag
    out per position for move generation; mask, position and the logits of the half-words that
    hold a move in, 96 edges out for the expansion), and the chain movegen -> evaluator ->
    expansion on one stream."""
    import torch
    from brokefish_amd.hip_impl import expand_edges, movegen
    out = []
    for nb in (256, 4096, 65536):
        bd, cd, rd, md = inputs[nb]
        policy, promo, value = model.forward_full(bd, cd, rd)
        gen = movegen(bd, cd)
        edges = expand_edges(policy, promo, value, md, bd, cd)
        iters = 50 if nb <= 4096 else 10

        def timed(fn):
            for _ in range(3):
                fn()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(iters):
                fn()
            e1.record()
            e1.synchronize()
            return e0.elapsed_time(e1) / iters
        t_gen = timed(lambda: movegen(bd, cd, out=gen))
        t_exp = timed(lambda: expand_edges(policy, promo, value, md, bd, cd, out=edges))
        t_chain = timed(lambda: model.forward_expand(bd, cd, rd, out=edges))
        gen_bytes = nb * (64 + 2 + 256 + 1)
        # the expansion reads a half-row of policy logits (32 fp16) only where a half-word of the mask
        # names a move: mask, position and value in, those half-rows, 96 edges and the counters out
        halves = int(((md & 0xFFFFFFFF) != 0).sum() + ((md >> 32) != 0).sum())
        exp_bytes = nb * (256 + 64 + 2 + 4) + 64 * halves + nb * (96 * 4 + 4 + 4 + 4 + 2)
        out.append({"batch": nb, "movegen_ms": t_gen, "movegen_positions_per_s": nb / t_gen * 1e3,
                    "movegen_GBps": gen_bytes / t_gen / 1e6, "movegen_frac_hbm": gen_bytes / (t_gen * 1e-3) / PEAK_HBM_BPS,
                    "expand_ms": t_exp, "expand_GBps": exp_bytes / t_exp / 1e6, "expand_frac_hbm": exp_bytes / (t_exp * 1e-3) / PEAK_HBM_BPS,
                    "chain_ms": t_chain})
    return out


def parity_report(net):
    """What is checked next to the number: a sample of the batch bit for bit against the C checker,
    and the prior-space distance to the int8 emulation as the reference reports it
    (brokefish/nn/validate.py:314-388: max |dp|, 95th percentile, top-1 moved, flip)."""
    import numpy as np
    import torch
    from brokefish_amd import encoder_impl, positions, validate
    from oracle import c_oracle, emulated
    sd = {k: v.detach() for k, v in net.state_dict().items()}
    b, c, r, m = positions.random_positions(128, plies=120, seed=1)
    bd, cd, rd, md = b.cuda(), c.cuda(), r.cuda(), m.cuda()
    model = encoder_impl("hip")(net, int8=True, out_dtype=torch.float32)
    got = [t.clone() for t in model.forward_masked(bd, cd, rd, md)]
    want = c_oracle.COracle(sd).forward(b.numpy(), c.numpy(), r.numpy(), mask=m.numpy())
    exact = all((g.cpu().numpy().view(np.int32) == want[k].view(np.int32)).all()
                for k, g in (("policy", got[0]), ("promo", got[1]), ("value", got[2]))) and \
        bool((got[3].cpu().numpy() == want["best"]).all())
    with torch.no_grad():
        emu = emulated.forward(sd, b, c, r, mode="int8")
    raw = [t.clone() for t in model.forward_full(bd, cd, rd)]
    d = validate.compare("kernel vs int8 emulation", tuple(t.cuda() for t in emu), raw, md, bd, cd)
    return {"positions": 128, "bit_exact_vs_c_checker": bool(exact), "masked_argmax_equal": bool((got[3].cpu().numpy() == want["best"]).all()),
            "prior_space_vs_int8_emulation": {k: v for k, v in d.as_dict().items() if k != "name"}}


if __name__ == "__main__":
    raise SystemExit(main())
