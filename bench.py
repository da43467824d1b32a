"""Headline benchmark: env-steps/sec of the 8192-env K-Bot-scale rollout on one MI355X.

A "step" is one control step of every env: observation (+noise) -> actor and critic MLPs (bf16 MFMA) -> action
sampling -> fused physics (4 substeps) -> termination + transition record + reset -> forward pass of the reset
envs; every `--rollout` steps the rewards and GAE kernels run over the recorded rollout.  Inputs are synthetic,
seeded, resident in HBM before the timed region.  Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E
BF16_PEAK_TFLOPS = 2500.0  # dense MFMA bf16
FP32_VALU_PEAK_TFLOPS = 157.3
# Untimed control steps every rollout of this file runs before its warm-up: the robots start on both feet, and it takes a
# few seconds of simulated time before falls, resets and airborne envs are in their steady proportions.  Independent of
# --warmup, so that a short timed window measures the same mixture as a long one.
PREROLL_STEPS = 240


def cpu_baseline(integrator: str, target_seconds: float = 12.0):
    """The oracle's C restatement of the control step (float32, OpenMP over envs) on this host's cores, on the same
    model (same integrator) as the GPU leg."""
    import numpy as np

    from ksim_amd import model as km
    from ksim_amd.configs import KBOT_TORQUE_LIMITS
    from oracle.dyn import Oracle

    from ksim_amd.configs import integrator_name

    m = km.kbot_scale_model(seed=1004, integrator=integrator)
    orc = Oracle(m.arrays(), np.float32)
    cores = min(16, os.cpu_count() or 1)
    N = 2048
    rng = np.random.default_rng(1004)
    block = orc.batch(N)
    for e in range(N):
        d = block[e]
        q = m.qpos0.copy()
        q[7:] += rng.uniform(-0.1, 0.1, m.nu)
        for i, v in enumerate(q):
            d.qpos[i] = v
        for b in range(m.nb):
            d.mass_scale[b] = rng.uniform(0.9, 1.1)
        d.friction = rng.uniform(0.4, 1.2)
    last = np.zeros((N, m.nu), dtype=np.float32)
    kp = np.tile(rng.uniform(20, 150, m.nu), (N, 1))
    kd = np.tile(rng.uniform(0.5, 1.5, m.nu), (N, 1))
    lat = np.zeros(N)

    def run(k):
        t0 = time.perf_counter()
        for _ in range(k):
            act = rng.normal(scale=0.1, size=(N, m.nu))
            orc.ctrl_step_batch(block, 4, 1, act, last, lat, None, kp, kd, KBOT_TORQUE_LIMITS, nthreads=cores)
        return time.perf_counter() - t0

    run(10)  # let the robots land on their feet so contacts are active, as in the GPU run
    t1 = run(2)
    k = max(2, int(target_seconds / max(t1 / 2, 1e-3)))
    t = run(k)
    return {"value": N * k / t, "unit": "env-steps/s", "cores": cores, "kind": "port",
            "sample": f"physics control step only (PD + 4 substeps, {integrator_name(m)}), {N} envs x {k} steps, "
                      f"float32 C restatement of the MJX path (not MJX), OpenMP over envs",
            "flops_per_env_step": oracle_flops_per_env_step(m, KBOT_TORQUE_LIMITS)}


def oracle_flops_per_env_step(m, ctrl_clip, envs: int = 32, settle: int = 10, counted: int = 4) -> float:
    """Floating-point operations of one control step (PD + 4 substeps) of one env, counted by running the oracle's C
    source with a scalar type that counts +, -, *, / and elementary functions as one operation each (dense algebra as the
    oracle writes it; the kernel skips structural zeros of the tree, so this is an upper bound on the useful work)."""
    import numpy as np

    from oracle.dyn import Oracle

    orc = Oracle(m.arrays(), np.float64, count_flops=True)
    rng = np.random.default_rng(1004)
    block = orc.batch(envs)
    for e in range(envs):
        q = m.qpos0.copy()
        q[7:] += rng.uniform(-0.1, 0.1, m.nu)
        for i, v in enumerate(q):
            block[e].qpos[i] = v
        for b in range(m.nb):
            block[e].mass_scale[b] = rng.uniform(0.9, 1.1)
        block[e].friction = rng.uniform(0.4, 1.2)
    last = np.zeros((envs, m.nu))
    kp = np.tile(rng.uniform(20, 150, m.nu), (envs, 1))
    kd = np.tile(rng.uniform(0.5, 1.5, m.nu), (envs, 1))
    for k in range(settle + counted):
        if k == settle:
            orc.flops_reset()
        orc.ctrl_step_batch(block, 4, 1, rng.normal(scale=0.1, size=(envs, m.nu)), last, np.zeros(envs), None, kp, kd,
                            ctrl_clip, nthreads=1)
    return orc.flops() / (envs * counted)


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--envs", type=int, default=8192)
    ap.add_argument("--rollout", type=int, default=32)
    ap.add_argument("--integrator", choices=("euler", "implicitfast"), default="euler",
                    help="velocity update of the headline rollout: semi-implicit Euler (what the benchmark configs name) or "
                         "implicitfast (what ksim's RLConfig selects); the other one is reported under 'other_integrator'")
    ap.add_argument("--only", choices=("mlp", "gae", "update", "kbot_update", "kbot_rollout", "kbot_iteration", "rollout", "iteration", "phases", "mfma"), default=None,
                    help="run one section alone and print its JSON (the command the counter runs under profiles/ use)")
    ap.add_argument("--mlp-rows", type=int, default=0, help="with --only mlp: a single row count instead of 8192 and 524288")
    ap.add_argument("--streams", type=int, default=2,
                    help="groups the envs are rolled out in, each on its own HIP stream (1: a single chain of launches)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also launch ks_copy_f32 on 64 Mi floats once: the known-size kernel for counter calibration")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch

    from ksim_amd import _lib, ppo
    from ksim_amd.configs import integrator_name, step_algorithmic_bytes

    if args.only == "phases":  # needs the -DKS_PROFILE build: python -m ksim_amd.csrc.build --profile
        from ksim_amd.csrc.build import PROFILE_LIB

        if not os.path.exists(PROFILE_LIB):
            sys.exit(f"{PROFILE_LIB} is not built: run `python -m ksim_amd.csrc.build --profile` first")
        _lib.LIB_PATH = PROFILE_LIB
    _lib.load()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    if args.traffic_probe:  # first, so that every --only section carries the calibration launch
        n = 64 * 1024 * 1024
        src, dst = torch.ones(n, device="cuda"), torch.empty(n, device="cuda")
        _lib.check(_lib.load().ks_copy_f32(_lib.current_stream(), n, _lib.ptr(src), _lib.ptr(dst)))
        torch.cuda.synchronize()
        del src, dst
    if args.only == "phases":
        print(json.dumps({"step_kernel_phases": step_kernel_phases(torch, args.integrator, args.envs),
                          "mlp_phases": mlp_phases(torch)}))
        return
    if args.only == "mfma":
        print(json.dumps({"mfma_yardstick": mfma_yardstick(torch)}))
        return
    if args.only == "mlp":
        print(json.dumps({"policy_mlp": mlp_rate(torch, rows=(args.mlp_rows,) if args.mlp_rows else (8192, 524288))}))
        return
    if args.only == "gae":
        print(json.dumps({"gae": gae_bandwidth(torch, ppo), "streaming": loss_and_reward_bandwidth(torch)}))
        return
    if args.only == "update":
        print(json.dumps({"ppo_update": ppo_update_rate(torch)}))
        return
    if args.only == "kbot_update":
        print(json.dumps({"kbot_update": kbot_update_rate(torch)}))
        return
    if args.only == "kbot_rollout":
        print(json.dumps({"kbot_rollout": kbot_rollout_rate(torch)}))
        return
    if args.only == "kbot_iteration":
        print(json.dumps({"kbot_iteration": kbot_iteration_rate(torch)}))
        return
    if args.only == "iteration":
        print(json.dumps({"ppo_iteration": ppo_iteration_rate(torch)}))
        return
    N = args.envs
    T = max(1, min(args.rollout, args.steps))  # the timed region holds whole rollouts, so rewards and GAE are inside it
    head = timed_rollout(torch, args.integrator, N, T, args.steps, args.warmup, args.streams)
    consts, elapsed, kernel_ms, ndone = (head[k] for k in ("consts", "elapsed", "kernel_ms", "ndone"))
    envs_per_launch = head["envs_per_launch"]
    head_stats = {k: head[k] for k in ("nefc_mean", "niter_mean", "in_contact")}
    m = consts.physics_model.model
    other = "implicitfast" if args.integrator == "euler" else "euler"
    if args.only == "rollout":  # the timed rollout alone: what the kernel-trace and counter runs of the step kernel profile
        print(json.dumps({"value": N * args.steps / elapsed, "ms_per_step": elapsed / args.steps * 1e3,
                          "step_kernel_ms": kernel_ms, "integrator": integrator_name(m), "num_envs": N, "rollout_length": T,
                          "streams": args.streams, "envs_per_step_launch": envs_per_launch,
                          "untimed_preroll_steps": PREROLL_STEPS, "episodes_finished_in_timed_region": ndone,
                          "constraint_rows_mean": head["nefc_mean"], "newton_iterations_mean": head["niter_mean"],
                          "envs_in_contact": head["in_contact"]}))
        return
    del head
    # The same rollout over a window long enough that filling and draining the two launch chains (about one control step
    # at each end of the bracketing synchronisations) no longer shows: the figure a training run sees.
    long_entry = None
    if args.steps < 200:
        lg = timed_rollout(torch, args.integrator, N, args.rollout, 200, 0, args.streams)
        long_entry = {"value": N * lg["steps"] / lg["elapsed"], "unit": "env-steps/s", "steps": lg["steps"],
                      "ms_per_step": lg["elapsed"] / lg["steps"] * 1e3, "step_kernel_ms": lg["kernel_ms"],
                      "rollout_length": args.rollout, "episodes_finished_in_timed_region": lg["ndone"]}
        del lg
    alt = timed_rollout(torch, other, N, T, max(T, min(args.steps, 2 * T)), min(args.warmup, T), args.streams)
    other_entry = {"integrator": integrator_name(alt["consts"].physics_model.model),
                   "value": N * alt["steps"] / alt["elapsed"], "unit": "env-steps/s", "steps": alt["steps"],
                   "ms_per_step": alt["elapsed"] / alt["steps"] * 1e3, "step_kernel_ms": alt["kernel_ms"]}
    del alt

    # The same workload as ONE chain of launches on one stream (all N envs per launch), and that chain captured once as a
    # HIP graph and replayed, which takes the host out of the loop.
    single = timed_rollout(torch, args.integrator, N, T, max(T, min(args.steps, 2 * T)), min(args.warmup, T), 1)
    env, ro = single["env"], single["ro"]
    single_entry = {"value": N * single["steps"] / single["elapsed"], "unit": "env-steps/s", "steps": single["steps"],
                    "ms_per_step": single["elapsed"] / single["steps"] * 1e3, "step_kernel_ms": single["kernel_ms"],
                    "envs_per_step_launch": N}
    graph = None
    if not args.traffic_probe:
        reps = max(1, args.steps // T)
        ro.unroll(env, graph=True)  # capture + first replay
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            rew = ro.unroll(env, graph=True)[1]
            ro.ppo_inputs(rew, 0.99, 0.95, normalize_advantages=True)
        torch.cuda.synchronize()
        g_elapsed = time.perf_counter() - t0
        assert torch.isfinite(env.physics_state.data.qpos).all(), "non-finite state after the graph replays"
        graph = {"value": N * reps * T / g_elapsed, "unit": "env-steps/s", "steps": reps * T,
                 "ms_per_step": g_elapsed / (reps * T) * 1e3,
                 "what": "the same control steps, rewards and GAE with each T-step rollout replayed from one HIP graph"}

    # GAE on rotating cfg-2 sized buffers (T=128, N=4096): larger than the caches in total
    gae = gae_bandwidth(torch, ppo)
    streaming = loss_and_reward_bandwidth(torch)
    mlp = mlp_rate(torch)
    mlp["mfma_yardstick"] = mfma_yardstick(torch)
    top = mlp["mfma_yardstick"]["all_cus_two_waves_per_simd"]["TFLOPs"]
    for key in ("rows_8192", "rows_524288"):
        mlp[key]["of_mfma_yardstick"] = mlp[key]["TFLOPs"] / top
    upd = ppo_update_rate(torch)
    kbot_upd = kbot_update_rate(torch)
    kbot_ro = kbot_rollout_rate(torch)
    kbot_it = kbot_iteration_rate(torch)
    iteration = ppo_iteration_rate(torch)

    obs_dim = consts.terms.obs_dim
    bytes_per_env = step_algorithmic_bytes(m, obs_dim, 1 + m.nb)
    achieved = bytes_per_env * envs_per_launch / (kernel_ms * 1e-3) / 1e9  # one launch steps the envs of one group
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "step_kernel_cfg4_hbm_traffic.txt")
    if os.path.exists(tpath):  # measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, see that file
        for ln in open(tpath):
            # counted on launches of 8192 envs and of 4096 envs (the two-stream groups): the figure of this run's shape
            key = "hbm_bytes_per_env_step_4096_env_launch=" if envs_per_launch <= 4096 else "hbm_bytes_per_env_step="
            if ln.startswith(key):
                traffic = float(ln.split("=", 1)[1]) * envs_per_launch
    valu = {}
    vpath = os.path.join(ROOT, "profiles", "step_kernel_cfg4_instruction_mix.txt")
    if os.path.exists(vpath):  # rocprofv3 --pmc SQ_* summary, see that file
        for ln in open(vpath):
            if ln.startswith("valu_"):
                k, v = ln.strip().split("=", 1)
                valu[k] = float(v)
    line = {
        "metric": "env-steps/sec, 8192-env humanoid rollout (1 GPU)", "value": N * args.steps / elapsed,
        "unit": "env-steps/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "cfg4: K-Bot-scale biped (free root + 20 hinges, 8 foot spheres), per-env friction/mass "
                               "randomisation, obs noise 0.01, reset on z<0.5, actor+critic 3x512 bf16 MLP, "
                               f"dt=0.005 x 4 substeps, Newton 8/8, {integrator_name(m)} integration; rewards + GAE after "
                               f"every {T} control steps inside the timed region; envs in {args.streams} independent "
                               f"group(s), one HIP stream each",
                   "integrator": integrator_name(m), "num_envs": N, "rollout_length": T, "substeps": 4,
                   "streams": args.streams, "envs_per_step_launch": envs_per_launch,
                   "obs_dim": obs_dim, "untimed_preroll_steps": PREROLL_STEPS,
                   "episodes_finished_in_timed_region": ndone,
                   "constraint_rows_mean": head_stats["nefc_mean"], "newton_iterations_mean": head_stats["niter_mean"],
                   "envs_in_contact": head_stats["in_contact"]},
        "roofline": {"bound": "hbm", "kernel": "step_kernel (fused control step)", "achieved": achieved,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                     "algorithmic_bytes_per_env_step": bytes_per_env, "kernel_ms": kernel_ms,
                     "envs_per_launch": envs_per_launch,
                     "valu_issue_fraction_profiled": valu.get("valu_issue_fraction"),
                     "valu_insts_per_env_step_profiled": valu.get("valu_insts_per_env_step"),
                     "counters_source": "traffic and valu_* are read from the committed rocprofv3 --pmc summaries under "
                                        "profiles/ (separate counter runs of this command), not re-measured in this run",
                     "note": "the fused step is bound by fp32 vector-ALU issue (~1e3 flop/byte; the profiled share of "
                             "cycles with a VALU instruction issuing is given beside); the HBM fraction is reported "
                             "against the bytes the engine contract obliges a step to move"},
        "same_rollout_200_steps": long_entry, "other_integrator": other_entry, "single_stream": single_entry,
        "gae": gae, "streaming": streaming, "policy_mlp": mlp, "ppo_update": upd, "kbot_update": kbot_upd, "kbot_rollout": kbot_ro, "kbot_iteration": kbot_it, "ppo_iteration": iteration, "graph_replay": graph,
    }
    if not args.no_cpu_baseline:
        base = cpu_baseline(args.integrator)
        flops = base.pop("flops_per_env_step")
        line["cpu_baseline"] = base
        rate = flops * envs_per_launch / (kernel_ms * 1e-3) / 1e12
        whole = flops * N / (elapsed / args.steps) / 1e12  # all groups together, per wall-clock control step
        line["roofline"]["fp32_valu"] = {
            "achieved": rate, "peak": FP32_VALU_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": rate / FP32_VALU_PEAK_TFLOPS,
            "flops_per_env_step": flops, "achieved_all_groups": whole, "frac_all_groups": whole / FP32_VALU_PEAK_TFLOPS,
            "what": "floating-point operations of one env's control step as the float64 oracle performs them (counted by "
                    "a build of its C source with a counting scalar type, 32 standing envs) x envs per launch / the "
                    "step kernel's measured duration; with several groups in flight a launch shares the chip with the "
                    "other group's, so 'all_groups' divides the flops of all envs by the wall-clock time of a control step"}
    print(json.dumps(line))


def timed_rollout(torch, integrator: str, N: int, T: int, steps: int, warmup: int, streams: int = 2,
                  preroll: int = PREROLL_STEPS) -> dict:
    """`preroll` + `warmup` untimed control steps, then exactly `steps` timed ones of the cfg 4 rollout built with `integrator`.
    The rollout slot restarts at 0 where the timed region begins, so it holds steps // T reward + GAE passes.
    `streams`: the N envs run as that many independent groups, each on its own HIP stream (1 = one launch chain)."""
    from ksim_amd.configs import kbot_rollout, kbot_split_rollout
    from ksim_amd.rewards import get_rewards

    if streams > 1:
        consts, envs, ro = kbot_split_rollout(num_envs=N, rollout_length=T, splits=streams, integrator=integrator)
    else:
        consts, env, ro, _ = kbot_rollout(num_envs=N, rollout_length=T, integrator=integrator)
    # time the dominant kernel (the fused physics control step) with events on the stream of each launch
    step_events: list = []
    orig_step = consts.engine.step

    def timed_step(*a, **kw):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        out = orig_step(*a, **kw)
        e1.record()
        step_events.append((e0, e1))
        return out

    def one_step(t: int) -> None:
        if streams > 1:
            ro.step_engine(envs, t)
            if t == T - 1:
                rews = []
                for part, st in zip(ro.parts, ro.streams):
                    with torch.cuda.stream(st):
                        rews.append(get_rewards(part.trajectory(), consts.rewards, want_components=False))
                ro.ppo_inputs(rews, 0.99, 0.95, normalize_advantages=True)  # joins the groups for the normalisation
        else:
            ro.step_engine(env, t)
            if t == T - 1:
                rew = get_rewards(ro.trajectory(), consts.rewards, want_components=False)
                ro.ppo_inputs(rew, 0.99, 0.95, normalize_advantages=True)

    parts = ro.parts if streams > 1 else [ro]
    states = envs if streams > 1 else [env]
    group_streams = ro.streams if streams > 1 else [torch.cuda.current_stream()]
    # episodes that end inside the timed region: each group adds up the done flags of a rollout's slots when the rollout is
    # complete (one small reduction per group and T steps, on the group's stream, no host synchronisation)
    finished = [torch.zeros((), dtype=torch.int64, device="cuda") for _ in parts]

    def count_finished(k: int) -> None:
        if k % T == T - 1 or k == steps - 1:
            for part, st, acc in zip(parts, group_streams, finished):
                with torch.cuda.stream(st):
                    acc += part.done[: k % T + 1].sum()

    if streams > 1:
        ro.fork()
    for k in range(preroll + warmup):
        one_step(k % T)
    count_finished(T - 1)  # the reduction's first launch loads its code object: not inside the timed region
    for acc in finished:
        acc.zero_()
    consts.engine.step = timed_step
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(steps):
        one_step(k % T)
        count_finished(k)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    consts.engine.step = orig_step
    kernel_ms = sum(a.elapsed_time(b) for a, b in step_events) / len(step_events)
    ndone = sum(int(f.item()) for f in finished)
    # what the solver is working on in this state of the simulation: constraint rows and Newton iterations of the last
    # substep of one more (untimed) control step
    nefc, niter, contact = [], [], []
    for part, e, st in zip(parts, states, group_streams):
        with torch.cuda.stream(st):
            stats = {k: torch.zeros(part.N, dtype=torch.int32, device="cuda") for k in ("nefc", "solver_niter")}
            consts.engine.step(part.action[0], consts.physics_model, e.physics_state, 1.0, e.seed + e.step, e.randomization_dict, stats=stats)
        torch.cuda.synchronize()
        nefc.append(stats["nefc"].float().mean().item())
        niter.append(stats["solver_niter"].float().mean().item())
        contact.append((stats["nefc"] > 0).float().mean().item())
    for e in states:
        assert torch.isfinite(e.physics_state.data.qpos).all(), "non-finite state after the benchmark"
    g = len(parts)
    return dict(consts=consts, env=states[0], ro=parts[0], elapsed=elapsed, kernel_ms=kernel_ms, ndone=ndone, steps=steps,
                envs_per_launch=N // streams, nefc_mean=sum(nefc) / g, niter_mean=sum(niter) / g, in_contact=sum(contact) / g)


def gae_bandwidth(torch, ppo, reps=8):
    """GAE GB/s through the C ABI on rotating buffer sets (larger in total than the caches), outputs preallocated."""
    from ksim_amd import _lib

    lib = _lib.load()
    out = {}
    for name, N, T, sets in (("cfg2_T128_N4096", 4096, 128, 32), ("large_T128_N65536", 65536, 128, 4)):
        g = torch.Generator(device="cuda")
        g.manual_seed(1002)
        bufs = [(torch.randn(N, T, device="cuda", generator=g), torch.randn(N, T, device="cuda", generator=g),
                 (torch.rand(N, T, device="cuda", generator=g) < 0.01).view(torch.uint8)) for _ in range(sets)]
        res = [torch.empty(N, T, device="cuda") for _ in range(3)]
        st = _lib.current_stream()

        def run(v, r, d):
            _lib.check(lib.ks_gae_bt(st, N, T, _lib.ptr(v), _lib.ptr(r), _lib.ptr(d), None, 0.99, 0.95, 0,
                                     _lib.ptr(res[0]), _lib.ptr(res[1]), _lib.ptr(res[2])))

        for b in bufs[:2]:
            run(*b)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            for b in bufs:
                run(*b)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / (reps * sets)
        nbytes = T * N * 21
        out[name] = {"layout": "(B,T) fp32, dones int8", "ms_per_call": ms, "achieved_GBps": nbytes / (ms * 1e-3) / 1e9,
                     "frac_of_hbm_peak": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "algorithmic_bytes": nbytes,
                     "buffer_sets": sets}
    # yardstick for cfg 2: a plain copy kernel that moves the same 11 MB per call (half read, half written), on buffers
    # rotated the same way; what it reaches is what a single launch of this size can reach on this machine
    n_copy = 4096 * 128 * 21 // 8
    cb = [(torch.randn(n_copy, device="cuda"), torch.empty(n_copy, device="cuda")) for _ in range(32)]
    for a, b in cb[:2]:
        _lib.check(lib.ks_copy_f32(_lib.current_stream(), n_copy, _lib.ptr(a), _lib.ptr(b)))
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        for a, b in cb:
            _lib.check(lib.ks_copy_f32(_lib.current_stream(), n_copy, _lib.ptr(a), _lib.ptr(b)))
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / (reps * len(cb))
    out["cfg2_T128_N4096"]["plain_copy_of_the_same_bytes"] = {"ms_per_call": ms, "achieved_GBps": n_copy * 8 / (ms * 1e-3) / 1e9}
    del cb
    # the rollout's own layout (T, N), with the success flags it carries: cfg 4 / cfg 5 shapes and a large one
    for name, N, T, sets in (("rollout_T32_N8192", 8192, 32, 64), ("rollout_T32_N16384", 16384, 32, 32),
                             ("large_T128_N65536_tn", 65536, 128, 4)):
        g = torch.Generator(device="cuda")
        g.manual_seed(1004)
        bufs = [(torch.randn(T, N, device="cuda", generator=g), torch.randn(T, N, device="cuda", generator=g),
                 (torch.rand(T, N, device="cuda", generator=g) < 0.01).view(torch.uint8),
                 torch.zeros(T, N, dtype=torch.uint8, device="cuda")) for _ in range(sets)]
        res = [torch.empty(T, N, device="cuda") for _ in range(3)]
        st = _lib.current_stream()

        def run_tn(v, r, d, sc):
            _lib.check(lib.ks_gae_tn(st, T, N, _lib.ptr(v), _lib.ptr(r), _lib.ptr(d), _lib.ptr(sc), 0.99, 0.95, 0,
                                     _lib.ptr(res[0]), _lib.ptr(res[1]), _lib.ptr(res[2])))

        for b in bufs[:2]:
            run_tn(*b)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            for b in bufs:
                run_tn(*b)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / (reps * sets)
        nbytes = T * N * 22
        out[name] = {"layout": "(T,N) fp32, dones and successes int8", "ms_per_call": ms,
                     "achieved_GBps": nbytes / (ms * 1e-3) / 1e9, "frac_of_hbm_peak": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "algorithmic_bytes": nbytes, "buffer_sets": sets}
    return out


def loss_and_reward_bandwidth(torch, reps=8, sets=16):
    """The other two streaming kernels of cfg 2 (T=128, N=4096) through the C ABI on rotating buffer sets: the per-element PPO
    loss terms with their mean, and the reward sum with the done / success reduction over the termination components."""
    import ctypes
    from ksim_amd import _lib

    lib = _lib.load()
    n, A, K, k = 4096 * 128, 1, 8, 4
    g = torch.Generator(device="cuda")
    g.manual_seed(1002)
    rn = lambda *shape: torch.randn(*shape, device="cuda", generator=g)  # noqa: E731
    st = _lib.current_stream()
    out = {}

    def timed(run, bufs):
        for b in bufs[:2]:
            run(*b)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            for b in bufs:
                run(*b)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / (reps * len(bufs))

    # PPO loss: reads advantages, targets, on / off log-probabilities and values, entropy (7 floats at A = 1); writes the
    # policy / value / KL / entropy terms per element (the reference returns them per element, ppo.py:447-492) and their mean
    params = _lib.KsPpoLossParams(0.2, 0.5, 0.008, 1e-3, 5.0, 1.0, 1)
    ws = torch.empty(1 << 16, dtype=torch.uint8, device="cuda")
    res = [torch.empty(n, device="cuda") for _ in range(4)]
    total = torch.empty((), device="cuda")
    bufs = []
    for _ in range(sets):
        on_lp = rn(n, A)
        bufs.append((rn(n), rn(n), on_lp, rn(n), on_lp + 0.05 * rn(n, A), rn(n), rn(n, A)))

    def run_loss(adv, tgt, on_lp, on_v, off_lp, off_v, ent):
        _lib.check(lib.ks_ppo_loss(st, n, A, params, _lib.ptr(adv), _lib.ptr(tgt), _lib.ptr(on_lp), _lib.ptr(on_v), _lib.ptr(off_lp),
                                   _lib.ptr(off_v), _lib.ptr(ent), _lib.ptr(res[0]), _lib.ptr(res[1]), _lib.ptr(res[2]), _lib.ptr(res[3]),
                                   _lib.ptr(total), _lib.ptr(ws)))

    ms = timed(run_loss, bufs)
    nbytes = n * 4 * (4 + 3 * A + 4)
    out["ppo_loss_cfg2"] = {"ms_per_call": ms, "achieved_GBps": nbytes / (ms * 1e-3) / 1e9, "frac_of_hbm_peak": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                            "algorithmic_bytes": nbytes, "bytes_per_element": 4 * (4 + 3 * A + 4), "buffer_sets": sets}
    del bufs

    # reward total + done / success: K reward components (f32) and k termination components (int8) per element
    scales = (ctypes.c_float * K)(*[0.5 + 0.1 * i for i in range(K)])
    tot, done, succ = torch.empty(n, device="cuda"), torch.empty(n, dtype=torch.uint8, device="cuda"), torch.empty(n, dtype=torch.uint8, device="cuda")
    bufs = [(rn(K, n), (torch.randint(-1, 2, (k, n), device="cuda", generator=g) * (torch.rand(k, n, device="cuda", generator=g) < 0.01)).to(torch.int8))
            for _ in range(sets)]

    def run_reward(comp, term):
        _lib.check(lib.ks_reward_total(st, n, K, _lib.ptr(comp), scales, 1, -5.0, 1, 5.0, _lib.ptr(tot), k, _lib.ptr(term), _lib.ptr(done), _lib.ptr(succ)))

    ms = timed(run_reward, bufs)
    nbytes = n * (4 * K + k + 6)
    out["reward_total_cfg2"] = {"ms_per_call": ms, "achieved_GBps": nbytes / (ms * 1e-3) / 1e9, "frac_of_hbm_peak": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                                "algorithmic_bytes": nbytes, "bytes_per_element": 4 * K + k + 6, "reward_components": K, "termination_components": k,
                                "buffer_sets": sets}
    return out


def ppo_update_rate(torch, reps=6):
    """One minibatch step of the policy update at benchmark config 5's shape: 2048 envs x T=32 rows through actor and
    critic (3x512 bf16), GAE, loss gradient, backward GEMMs, optimiser chain."""
    from ksim_amd.mlp import random_mlp
    from ksim_amd.ppo_update import GaussianMlpPolicy, PPOUpdateConfig, get_ppo_variables, single_step

    Tn, b, od, A = 32, 2048, 68, 20
    actor, _, _ = random_mlp((od, 512, 512, 512, A), 0)
    critic, _, _ = random_mlp((od, 512, 512, 512, 1), 1)
    pol = GaussianMlpPolicy(actor=actor, critic=critic, log_std=torch.full((A,), -1.0, device="cuda"))
    pol.train_init()
    cfg = PPOUpdateConfig()
    g = torch.Generator(device="cuda")
    g.manual_seed(0)
    obs = torch.randn(Tn, b, od, device="cuda", generator=g)
    act = torch.randn(Tn, b, A, device="cuda", generator=g) * 0.3
    rew = torch.randn(Tn, b, device="cuda", generator=g)
    done = torch.rand(Tn, b, device="cuda", generator=g) < 0.02
    succ = torch.zeros_like(done)
    on_lp, on_v, _, _ = get_ppo_variables(pol, obs.reshape(-1, od), obs.reshape(-1, od), act.reshape(-1, A))
    on_lp, on_v = on_lp.view(Tn, b, A).clone(), on_v.view(Tn, b).clone()
    for _ in range(2):
        single_step(pol, cfg, obs, obs, act, rew, done, succ, on_lp, on_v)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        single_step(pol, cfg, obs, obs, act, rew, done, succ, on_lp, on_v)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / reps
    flops = 3 * (actor.flops_per_row() + critic.flops_per_row()) * Tn * b
    return {"rows": Tn * b, "ms_per_minibatch_step": ms, "TFLOPs": flops / ms / 1e9,
            "mfma_utilisation": flops / ms / 1e9 / (BF16_PEAK_TFLOPS),
            "what": "forward + backward (3x the forward flops) of actor and critic 68-3x512-{20,1} bf16, GAE, loss "
                    "gradient and optimiser chain on 2048 envs x 32 steps"}


def kbot_rollout_rate(torch, preroll=200, steps=200):
    """Rollout rate of the K-Bot-scale env with the K-Bot example's recurrent policy (`configs.kbot_lstm_rollout`: LSTM actor
    and critic 2 x 128 in fp32, filtered mean | deviation head, 4096 envs), after `preroll` untimed control steps."""
    from ksim_amd.configs import kbot_lstm_rollout

    consts, env, ro, _ = kbot_lstm_rollout()
    for k in range(preroll):
        ro.step_engine(env, k % ro.T)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(steps):
        ro.step_engine(env, k % ro.T)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    assert torch.isfinite(ro.values).all() and torch.isfinite(env.actor_carry).all()
    return {"num_envs": ro.N, "untimed_preroll_steps": preroll, "steps": steps, "ms_per_step": dt * 1e3, "value": ro.N / dt,
            "unit": "env-steps/s",
            "what": "control steps of 4096 envs with the K-Bot example's LSTM actor and critic (2 x 128, fp32) in the loop, "
                    "one chain of launches with the critic on a side stream"}


def kbot_iteration_rate(torch, reps=2):
    """Whole iterations of the K-Bot example's task shape (examples/kbot/train.py:1754-1757): a rollout of 4096 envs x 100
    control steps with the LSTM actor and critic in the loop, rewards, then the update: the on-policy pass replayed from the
    recorded carries, 3 passes x 8 minibatches of 512 envs through both networks with the filter and the mirrored pass."""
    import numpy as np

    from ksim_amd import ppo_update as pu
    from ksim_amd.configs import kbot_lstm_rollout

    consts, env, ro, _ = kbot_lstm_rollout()
    rng = np.random.default_rng(11)
    K = consts.terms.obs_dim
    operm, osign = list(rng.permutation(K)), list(rng.choice([-1.0, 1.0], K))
    aperm, asign = pu.kbot_mirror_joints()
    h = consts.head
    policy = pu.RecurrentHeadPolicy(consts.actor, consts.critic, h.min_std, h.max_std, h.var_scale, h.mean_bias, lowpass=h.lowpass,
                                    mirror=pu.MirrorSpec(operm, osign, operm, osign, aperm, asign))
    policy.train_init()
    cfg = pu.PPOUpdateConfig(batch_size=512, num_passes=3, learning_rate=3e-4, actor_mirror_loss_scale=1.0, critic_mirror_loss_scale=0.5)

    def iteration(seed: int):
        traj, rew = ro.unroll(env)
        torch.cuda.synchronize()
        t_roll = time.perf_counter()
        out = pu.update_model_recurrent(policy, cfg, traj.obs["noisy_obs"], traj.obs["obs"], traj.action, rew.total, traj.done,
                                        traj.success, ro.actor_carry0, ro.critic_carry0, ro.fresh, seed=seed, lpf0=ro.lpf_carry0)
        return t_roll, out

    for k in range(2):  # the first two rollouts also take the robots from their initial stance to falls and resets
        iteration(k)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    roll = 0.0
    for k in range(reps):
        torch.cuda.synchronize()  # so that the rollout's share does not include the tail of the previous update
        ts = time.perf_counter()
        t_roll, out = iteration(2 + k)
        roll += t_roll - ts
    torch.cuda.synchronize()
    elapsed = (time.perf_counter() - t0) / reps
    assert all(torch.isfinite(o["grad_norm"]).all() for o in out) and torch.isfinite(env.actor_carry).all()
    n = ro.N * ro.T
    return {"num_envs": ro.N, "rollout_length": ro.T, "transitions": n, "minibatch_envs": cfg.batch_size, "num_passes": cfg.num_passes,
            "minibatch_steps": len(out), "s_per_iteration": elapsed, "transitions_per_s": n / elapsed, "rollout_s": roll / reps,
            "update_s": elapsed - roll / reps,
            "what": "rollout of 4096 envs x 100 steps with the K-Bot example's LSTM policy, rewards, on-policy replay and 24 minibatch "
                    "steps with filter gradient and mirror losses; host wall-clock per iteration"}


def kbot_update_rate(torch, reps=4):
    """One minibatch step of the K-Bot task as shipped (examples/kbot/train.py:80-95, 1287-1310, 1754-1757): LSTM actor
    65 -> 2 x 128 -> 40 (means | deviations of 20 joints) and LSTM critic 475 -> 2 x 128 -> 1 in float32, 512 envs x 100
    control steps per minibatch, the one-pole low-pass on the biased means with its state in the carry, and the second pass
    of both networks over the mirrored observations from their own carries with the two mirror losses."""
    import numpy as np

    from ksim_amd import ppo_update as pu
    from ksim_amd.actions import LowPass
    from ksim_amd.mlp import MLP
    from ksim_amd.recurrent import LSTMCell, RecurrentNetwork

    rng = np.random.default_rng(7)
    Tn, b, Ia, Ic, H, nu = 100, 512, 65, 475, 128, 20

    def make(I, out_dim):
        proj = (rng.normal(size=(H, I)) / np.sqrt(I), rng.normal(size=H) * 0.1)
        cells = [LSTMCell(rng.normal(size=(4 * H, H)) / np.sqrt(H), rng.normal(size=(4 * H, H)) / np.sqrt(H),
                          rng.normal(size=4 * H) * 0.1, dtype="f32") for _ in range(2)]
        out = MLP([rng.normal(size=(out_dim, H)) / np.sqrt(H)], [rng.normal(size=out_dim) * 0.1], activation="none", dtype="f32")
        return RecurrentNetwork(proj, cells, out, dtype="f32")

    actor, critic = make(Ia, 2 * nu), make(Ic, 1)
    sp = lambda n: (list(rng.permutation(n)), list(rng.choice([-1.0, 1.0], n)))  # noqa: E731
    (pa, sa), (pc, sc), (pj, sj) = sp(Ia), sp(Ic), sp(nu)
    t32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.float32, device="cuda")  # noqa: E731
    policy = pu.RecurrentHeadPolicy(actor, critic, 0.01, 1.0, 0.5, t32(rng.normal(size=nu) * 0.1),
                                    mirror=pu.MirrorSpec(pa, sa, pc, sc, pj, sj), lowpass=LowPass(0.02, 10.0, obs_bias=(Ia - 11, 10, 10)))
    policy.train_init()
    cfg = pu.PPOUpdateConfig(batch_size=b, actor_mirror_loss_scale=1.0, critic_mirror_loss_scale=0.5)
    g = torch.Generator(device="cuda")
    g.manual_seed(0)
    r = lambda *s: torch.randn(*s, device="cuda", generator=g)  # noqa: E731
    aobs, cobs, act, rew = r(Tn, b, Ia), r(Tn, b, Ic), r(Tn, b, nu) * 0.3, r(Tn, b)
    fresh = (torch.rand(Tn, b, device="cuda", generator=g) < 0.01).to(torch.uint8)
    done = torch.roll(fresh, -1, 0)
    done[-1] = 0
    succ = torch.zeros_like(done)
    on_lp, on_v = r(Tn, b, nu) * 0.1 - 1.0, r(Tn, b) * 0.1
    carry = lambda: r(2, 2, b, H) * 0.3  # noqa: E731
    args = (aobs, cobs, act, rew, done, succ, on_lp, on_v, carry(), carry(), fresh, r(b, nu) * 0.1,
            pu.MirrorCarries(carry(), carry(), r(b, nu) * 0.1))
    out = None
    for _ in range(2):
        out = pu.single_step_recurrent(policy, cfg, *args)
    assert torch.isfinite(out["grad_norm"]).all()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(reps):
        pu.single_step_recurrent(policy, cfg, *args)
    e1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / reps
    ms = e0.elapsed_time(e1) / reps
    return {"minibatch_envs": b, "rollout_steps": Tn, "mirrored_columns": b, "ms_per_minibatch_step": ms, "host_ms_per_minibatch_step": wall * 1e3,
            "transitions_per_s": Tn * b / (ms * 1e-3),
            "what": "K-Bot task minibatch step: LSTM actor 65-2x128-40 and critic 475-2x128-1 (float32) through 100 steps for 512 envs "
                    "and their 512 mirror images in one pass, low-pass filter with its gradient through time, PPO + mirror losses, "
                    "backward through time, global-norm clip and Adam"}


STEP_PHASES = ("actuator + reload of constants", "forward kinematics", "com / cinert / cdof", "composite inertia + M",
               "velocities + RNE bias", "M rows / smooth force", "contacts", "Cholesky(M) + solve", "Jacobian rows",
               "warm start + cost", "constraint update", "Hessian JtDJ", "Cholesky(H) + solve", "line search", "-",
               "integration")


def step_kernel_phases(torch, integrator: str, N: int, steps: int = 30) -> dict:
    """Clock cycles (s_memtime, 100 MHz) that one env's wavefront spends in each phase of a control step (4 substeps), mean
    over the envs of the benchmark's standing K-Bot-scale robots; read from the profiling build of the library."""
    import numpy as np

    from ksim_amd import model as km
    from ksim_amd import physics

    m = km.kbot_scale_model(seed=1004, integrator=integrator)
    dm = physics.DeviceModel(m)
    rng = np.random.default_rng(0)
    t = lambda a: torch.tensor(a, dtype=torch.float32, device="cuda").contiguous()  # noqa: E731
    z = lambda *s, **k: torch.zeros(*s, device="cuda", **k)  # noqa: E731
    qpos = np.tile(m.qpos0, (N, 1))
    qpos[:, 7:] += rng.uniform(-0.1, 0.1, (N, m.nu))
    buf = dict(qpos=t(qpos), qvel=z(N, m.nv), qacc_warmstart=z(N, m.nv), time=z(N), last_ctrl=z(N, m.nu),
               action=t(rng.uniform(-0.1, 0.1, (N, m.nu))), kp=t(rng.uniform(20, 150, m.nu)), kd=t(rng.uniform(0.5, 1.5, m.nu)),
               ctrl_clip=t(np.full(m.nu, 80.0)), friction=t(rng.uniform(0.4, 1.2, N)), mass_scale=t(rng.uniform(0.9, 1.1, (N, m.nb))),
               xpos=z(N, m.nb * 3), xquat=z(N, m.nb * 4), solver_niter=z(N, dtype=torch.int32), nefc=z(N, dtype=torch.int32),
               dbg_M=z(N, m.nv * m.nv))
    for _ in range(steps):
        physics.control_step(dm, buf, substeps=4)
    torch.cuda.synchronize()
    p = buf["dbg_M"][:, :16].cpu().numpy().astype(np.float64)
    total = float(p.sum(1).mean())
    return {"num_envs": N, "integrator": integrator, "lds_bytes_per_env": dm.lds_bytes, "cycles_per_control_step": total,
            "newton_iterations_mean": float(buf["solver_niter"].float().mean().item()),
            "constraint_rows_mean": float(buf["nefc"].float().mean().item()),
            "phases": {n: {"cycles": float(p[:, i].mean()), "share": float(p[:, i].mean()) / total}
                       for i, n in enumerate(STEP_PHASES) if n != "-"}}


def mlp_phases(torch, rows=524288) -> dict:
    """Where a workgroup of the whole-network MLP kernel (128-row tile, cfg 4 actor) spends its time: wall-clock stamps
    (100 MHz counter) of wavefront 0 between the phases of each layer, mean over the workgroups of one launch; read from
    the profiling build of the library, which takes the stamp buffer's address from KS_MLP_PROF_PTR."""
    import numpy as np

    from ksim_amd.configs import _net

    actor = _net((68, 512, 512, 512, 20), np.random.default_rng(1004), last_scale=0.1)
    blocks = (rows + 127) // 128
    prof = torch.zeros(blocks * 32, dtype=torch.int64, device="cuda")
    os.environ["KS_MLP_PROF_PTR"] = hex(prof.data_ptr())
    x, y = torch.randn(rows, actor.in_dim, device="cuda"), torch.empty(rows, actor.out_dim, device="cuda")
    for _ in range(3):
        actor(x, out=y)
    torch.cuda.synchronize()
    del os.environ["KS_MLP_PROF_PTR"]
    p = prof.cpu().numpy().reshape(blocks, 32)[:, :14].astype(np.float64)
    d = (p[:, 1:] - p[:, :-1]) * 10.0  # ns
    names = ["stage_input"] + [f"layer{l}_{w}" for l in range(4) for w in ("mfma_loop", "wait", "epilogue")]
    return {"rows": rows, "workgroups": blocks, "tile_rows": 128,
            "us_per_workgroup": float((p[:, 13] - p[:, 0]).mean() * 0.01),
            "launch_span_us": float((p[:, 13].max() - p[:, 0].min()) * 0.01),
            "phases_ns": {n: float(d[:, i].mean()) for i, n in enumerate(names)},
            "what": "mfma_loop: weight fragments from L2 + MFMAs over the layer's K; wait: the barrier before the activation "
                    "tile in LDS may be overwritten; epilogue: bias, activation, bf16 pack, write of the tile to LDS (last "
                    "layer: to memory)"}


def ppo_iteration_rate(torch, reps=3):
    """Whole training iterations at benchmark config 5's size: a 16384-env x 32-step rollout, discriminator scoring of the
    trajectory's motion frames, rewards with the AMP term, GAE and the on-policy pass, then 4 passes x 8 minibatches of
    2048 envs of actor / critic forward + backward + optimiser, with a discriminator step after each."""
    from ksim_amd.configs import kbot_ppo_iteration
    from ksim_amd.train_step import rl_train_loop_step

    consts, env, ro, policy, cfg, setup = kbot_ppo_iteration()
    gen = torch.Generator().manual_seed(0)
    rl_train_loop_step(ro, env, policy, cfg, amp=setup, generator=gen)  # warm-up: workspaces, optimiser state
    torch.cuda.synchronize()
    parts = {"rollout": 0.0, "update": 0.0}
    t0 = time.perf_counter()
    for _ in range(reps):
        out = rl_train_loop_step(ro, env, policy, cfg, amp=setup, generator=gen)
    torch.cuda.synchronize()
    elapsed = (time.perf_counter() - t0) / reps
    assert torch.isfinite(out["rewards"].total).all() and torch.isfinite(policy.log_std).all()
    # the rollout's share, timed alone on the same state
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for t in range(ro.T):
        ro.step_engine(env, t, 1.0, None)
    torch.cuda.synchronize()
    parts["rollout"] = time.perf_counter() - t0
    parts["update"] = elapsed - parts["rollout"]
    n = ro.N * ro.T
    return {"num_envs": ro.N, "rollout_length": ro.T, "transitions": n, "num_passes": cfg.num_passes,
            "minibatch_envs": cfg.batch_size, "minibatch_steps": len(out["steps"]), "discriminator": setup.disc.dims,
            "s_per_iteration": elapsed, "transitions_per_s": n / elapsed, "iterations_per_s": 1.0 / elapsed,
            "rollout_s": parts["rollout"], "postprocess_and_update_s": parts["update"],
            "what": "one rl_train_loop_step: rollout, discriminator scoring, rewards + GAE, 32 actor/critic minibatch steps "
                    "(bf16 3x512) each followed by a discriminator step (71-256-256-1); host wall-clock per iteration"}


def mfma_yardstick(torch, iters=20000):
    """What a loop of nothing but 32x32x16 bf16 MFMAs on register operands reaches on this GPU (`ks_mfma_yardstick`): the
    ceiling of any kernel built on that instruction, at the clock the part sustains under matrix load.  One wavefront per
    SIMD (256 workgroups of four) and two per SIMD (512), the occupancy of the whole-network MLP kernel."""
    from ksim_amd import _lib

    lib = _lib.load()
    out = {}
    for name, wgs in (("one_cu", 1), ("all_cus_one_wave_per_simd", 256), ("all_cus_two_waves_per_simd", 512)):
        sums = torch.empty(wgs * 256, device="cuda")
        stamps = torch.zeros(wgs * 2, dtype=torch.int64, device="cuda")
        _lib.check(lib.ks_mfma_yardstick(_lib.current_stream(), wgs, 200, _lib.ptr(sums), _lib.ptr(stamps)))  # warm-up
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        _lib.check(lib.ks_mfma_yardstick(_lib.current_stream(), wgs, iters, _lib.ptr(sums), _lib.ptr(stamps)))
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1)
        st = stamps.view(wgs, 2).double()
        n_mfma = iters * 8
        cyc, ticks = st[:, 0].mean().item(), st[:, 1].mean().item()
        tf = wgs * 4 * n_mfma * 32768.0 / (ms * 1e-3) / 1e12
        out[name] = {"workgroups": wgs, "ms": ms, "TFLOPs": tf, "of_nominal_bf16_peak": tf / BF16_PEAK_TFLOPS,
                     "shader_cycles_per_mfma_per_wave": cyc / n_mfma, "shader_clock_MHz_under_load": cyc / (ticks * 10.0) * 1e3}
    out["what"] = ("a loop of v_mfma_f32_32x32x16_bf16 only, 8 independent accumulator tiles per wavefront, operands in registers; "
                   "the clock is the ratio of the shader-cycle counter to the constant 100 MHz counter over the loop")
    return out


def mlp_rate(torch, rows=(8192, 524288), reps=20):
    """Forward pass of the cfg 4 actor (68 -> 3 x 512 -> 20, bf16 operands, fp32 accumulate) alone, at the rollout's
    row count and at a whole cfg 5 rollout's."""
    import numpy as np

    from ksim_amd.configs import _net

    actor = _net((68, 512, 512, 512, 20), np.random.default_rng(1004), last_scale=0.1)

    class _C:  # keeps the loop below reading like the rollout's call
        pass

    consts = _C()
    consts.actor = actor
    out = {}
    for M in rows:
        x = torch.randn(M, consts.actor.in_dim, device="cuda")
        y = torch.empty(M, consts.actor.out_dim, device="cuda")
        consts.actor(x, out=y)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            consts.actor(x, out=y)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / reps
        tf = consts.actor.flops_per_row() * M / (ms * 1e-3) / 1e12
        out[f"rows_{M}"] = {"ms": ms, "TFLOPs": tf, "mfma_utilisation": tf / BF16_PEAK_TFLOPS}
    out["net"] = "actor " + "x".join(str(d) for d in consts.actor.dims) + " bf16, fp32 accumulate"
    return out


if __name__ == "__main__":
    main()
