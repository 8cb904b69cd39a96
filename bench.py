"""Headline benchmark: env-steps/s of the batched articulation step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 1..6] [--envs 4096] [--mode eager|graph] [--only]

One "step" is one pass of the whole pipeline (FK, dynamics, contacts, block-descent solve, integration, FK) over
every environment of the batch, state resident in HBM.  Every timed step starts from the same seeded batch: the
state is put back by a device-side checkpoint restore INSIDE the timed region, so the figure is the cost of a step
on the published input distribution and does not drift with the trajectory.  (Left alone the trajectory is no
workload: the seeded torques act without change on joints that have no damping, velocities pass 10^3 rad/s within
ten steps and leave the fp32 range within a few dozen, in the library and in the CPU oracle alike, and a step over
such environments costs next to nothing.)  Prints ONE JSON line."""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

HBM_PEAK_GBPS = 8000.0
DOMINANT_OP = "BlockDescentSolve"
DOMINANT_KERNEL = "BlockDescentTileKernel"
SOLVER_SOURCES = ("nuka-physics_amd/csrc/ops_solver_kernel.h", "nuka-physics_amd/csrc/ops_solver.hip")


def solver_source_digest():
    """Names the dominant kernel's source as it stands: a counter summary is quoted only for the source it was taken on."""
    import hashlib
    digest = hashlib.sha256()
    for relative in SOLVER_SOURCES:
        with open(os.path.join(ROOT, relative), "rb") as handle:
            digest.update(handle.read())
    return digest.hexdigest()[:16]


def profiled_figures(name, envs):
    """What this script cannot measure itself - HBM bytes per launch of the dominant kernel and its instruction issue,
    from rocprofv3 --pmc runs - read from the committed summary of this workload (its `figures:` line), with the file it
    comes from and whether the kernel source is still the one the counters were taken on.  None without a summary."""
    relative = os.path.join("profiles", f"counters_{name}_{envs}.txt")
    try:
        with open(os.path.join(ROOT, relative)) as handle:
            lines = [line for line in handle if line.startswith("figures: ")]
    except OSError:
        return None
    if not lines:
        return None
    figures = json.loads(lines[-1][len("figures: "):])
    figures["from"] = relative
    figures["taken_on_this_source"] = figures.get("solver_source_sha256") == solver_source_digest()
    return figures


def algorithmic_bytes(nl, nv, nc, floating):
    """Bytes per env-step the step must move at least: state in/out (tier A) plus the fields the seam keeps in
    HBM once per step - packed M, packed L.D, bias, contact Jacobians - written once and read once (tier B)."""
    nj, f = nl - 1, 1 if floating else 0
    tier_a = 4 * ((3 * nj + 13 * f) + (nv + nj + nv + 7 * f + 7 * nl + 3 * nc + 2 * nc + 1))
    tier_b = 8 * (nv * (nv + 1) + nv + 3 * nc * nv)
    return tier_a, tier_a + tier_b


def solver_bytes(nv, nc):
    """The solve's share of that figure: it reads packed M, packed L.D, the contact Jacobians and the free velocity,
    and writes the velocity and the impulses."""
    return 4 * (nv * (nv + 1) + 3 * nc * nv + 2 * nv + 3 * nc)


def scene_run(nk, args):
    """Not the headline: a scene file's robot (MJCF or URDF, damped and driven joints) left to itself.  The batch
    settles for --settle steps from the authored pose with a small random push per environment, then --steps
    free-running steps are timed; environments that are flagged or not finite are counted, not hidden."""
    import numpy as np
    flags = nk.SCENE_GROUND_PLANE | nk.SCENE_PLANE_CONTACTS_ONLY if args.scene.endswith(".urdf") else 0
    if args.native_laws:            # an MJCF file's contacts and joint rows under the native laws instead of MuJoCo's
        flags |= nk.SCENE_NATIVE_CONTACT_LAW | nk.SCENE_NATIVE_JOINT_LAW
    scene = nk.Scene(args.scene, flags)
    E = args.envs or 4096
    device = nk.Device(0)
    world = nk.World(device, scene, nk.abi.world_desc(E, 0.0, vel_iters=8))
    nl = scene.link_count
    twist = np.zeros((E, nl, 6), np.float32)
    twist[:, 0] = np.random.default_rng(11).normal(0, 0.3, (E, 6))
    template = scene.to_c()[0]
    if template.free_body:          # a lone free body's state is its own row of the per-body velocity fields
        nb = template.body_count
        own = int(np.argmax(np.ctypeslib.as_array(template.body_role, shape=(nb,)) == nk.abi.ROLE_LINK_BODY))
        for name, part in (("body_linear_velocity", twist[:, 0, 3:]), ("body_angular_velocity", twist[:, 0, :3])):
            values = np.zeros((E, nb, 3), np.float32)
            values[:, own] = part
            world.upload(name, values)
    else:
        world.upload("link_velocity", twist)
    if args.base_height > 0.0:
        base = world.download("base_pose").reshape(E, 7).copy()
        base[:, 2] = args.base_height
        world.upload("base_pose", base)
    world.set_execution_mode(args.mode == "graph")
    world.step(args.settle)
    world.synchronize()
    start = time.perf_counter()
    world.step(args.steps)
    world.synchronize()
    wall_ms = (time.perf_counter() - start) * 1e3 / args.steps
    event_ms = world.time_steps(args.steps) / args.steps
    world.set_execution_mode(False)
    per_op = {}
    for name, ms in world.profile_ops(min(args.steps, 50)):
        per_op[name] = per_op.get(name, 0.0) + ms
    failed = int(((world.download("env_status") != 0) | ~np.isfinite(world.download("qdot").reshape(E, -1)).all(1)).sum())
    sweeps = world.download("vbd_velocity_sweep_count")
    result = {
        "metric": "env-steps/sec", "value": E * 1e3 / wall_ms, "unit": "env-steps/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.settle, "ms_per_step": wall_ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{os.path.basename(args.scene)}: {nl} links, {world.dof} DoF, {world.info.contact_slots_per_env} contact slots, "
                               f"{E} envs, free-running after {args.settle} settling steps" + (", native contact and joint laws" if args.native_laws else ""),
                   "envs": E, "execution": args.mode,
                   "event_ms_per_step": event_ms, "failed_envs": failed, "contacts_mean": float(world.download("contact_count").mean()),
                   "sweeps_mean": float(sweeps.mean()), "envs_using_every_sweep": int((sweeps == sweeps.max()).sum())},
        "per_op_ms": {k: round(v, 4) for k, v in per_op.items() if v >= 0.001},
    }
    world.close()
    device.close()
    print(json.dumps(result))


def cpu_baseline(nk, cfg, desc, budget_s=12.0):
    """The CPU oracle (a restatement of the reference algorithm, OpenMP over environments) on the same workload, on a
    bounded sample: at most 4096 environments of the seeded batch, stepped from the seeded state for budget_s."""
    oracle_py = entry.load_oracle()
    threads = min(16, os.cpu_count() or 1)
    E = min(cfg.env_count, 4096)
    desc = nk.abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters)
    world = oracle_py.OracleWorld(cfg.template, desc, threads=threads)
    state = cfg.state(E)
    world.set_state(state)
    world.step()                      # first touch of every page
    start = time.perf_counter()
    steps = 0
    while time.perf_counter() - start < budget_s:
        world.set_state(state)        # every step from the seeded batch, as on the GPU
        world.step()
        steps += 1
    elapsed = time.perf_counter() - start
    world.close()
    return {"value": E * steps / elapsed, "unit": "env-steps/s", "cores": threads, "kind": "port",
            "sample": f"{steps} steps of the first {E} environments of the same seeded batch in {elapsed:.1f} s, gcc -O2 -fopenmp"}


def apply_contact_law(nk, cfg, law):
    """`native` keeps the configuration as published; `elliptic` / `pyramidal` give every contact profile the MuJoCo law
    with that cone (the contact law of an imported MJCF file)."""
    if law == "native":
        return
    for profile in cfg.template.profiles:
        profile["law"] = nk.abi.LAW_MUJOCO
    cfg.template.contact_cone = nk.abi.CONE_ELLIPTIC if law == "elliptic" else nk.abi.CONE_PYRAMIDAL


def measure(nk, device, index, envs, steps, warmup, mode, cpu_budget_s, law="native"):
    """One configuration: warm-up, the timed steps (wall clock around back-to-back submissions and one final
    synchronisation), device events on the launch stream, per-op device times, and what the batch did - live
    contacts, sweeps used, environments at the sweep cap, environments that raised a status bit."""
    import numpy as np
    cfg = nk.synthetic.config(index, envs or None)
    apply_contact_law(nk, cfg, law)
    E = cfg.env_count
    desc = nk.abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters)
    world = nk.World(device, cfg.template, desc)
    world.set_state(cfg.state())
    world.set_execution_mode(mode == "graph")

    seeded = world.checkpoint()
    world.step_from(seeded, warmup)
    world.synchronize()
    start = time.perf_counter()
    world.step_from(seeded, steps)
    world.synchronize()
    wall_ms = (time.perf_counter() - start) * 1e3 / steps
    event_ms = world.time_steps(steps, seeded) / steps            # device events on the world's own stream

    nl, nv, solver_width = world.link_count, world.dof, world.info.solver_width
    nc = world.info.contact_slots_per_env
    batch = {"failed_envs": int((world.download("env_status") != 0).sum())}
    if world.rows_per_env:
        contacts, sweeps = world.download("contact_count"), world.download("vbd_velocity_sweep_count")
        batch.update(contacts_mean=float(contacts.mean()), contacts_max=int(contacts.max()), sweeps_mean=float(sweeps.mean()),
                     envs_at_sweep_cap=int((sweeps >= cfg.vel_iters).sum()), sweep_cap=cfg.vel_iters)

    # per-op durations with device events on the launch stream (eager dispatch), for the dominant kernel
    world.set_execution_mode(False)
    per_op = {}
    for name, ms in world.profile_ops(min(steps, 50), seeded):
        per_op[name] = per_op.get(name, 0.0) + ms
    dominant_ms = per_op.get(DOMINANT_OP, 0.0)
    tier_a, b_alg = algorithmic_bytes(nl, nv, nc, cfg.floating)
    if world.rows_per_env == 0 or dominant_ms == 0.0:             # contact-free worlds: dynamics is the step
        kernel, kernel_ms, kernel_bytes = "ArticulationDynamicsKernel", per_op.get("ArticulationDynamics", 0.0), 8 * (nv * (nv + 1) + nv) + 4 * (3 * (nl - 1) + 2 * nv)
    else:
        kernel, kernel_ms, kernel_bytes = DOMINANT_KERNEL, dominant_ms, solver_bytes(nv, nc)
    achieved = kernel_bytes * E / (kernel_ms * 1e-3) / 1e9 if kernel_ms > 0 else 0.0
    survey_gbps = b_alg * E / (kernel_ms * 1e-3) / 1e9 if kernel_ms > 0 else 0.0   # the whole step's bytes over the kernel's time
    step_gbps = b_alg * E / (wall_ms * 1e-3) / 1e9
    profiled = profiled_figures(cfg.name, E) if kernel == DOMINANT_KERNEL else None
    traffic = profiled.pop("traffic_bytes_per_launch", None) if profiled else None
    if profiled and not profiled["taken_on_this_source"]:
        traffic = None                                            # counters of an older kernel say nothing of this one
    blocks_per_cu = world.info.solver_blocks_per_cu
    live = ""
    if "contacts_mean" in batch:
        live = (f"; live contacts {batch['contacts_mean']:.1f} of {nc} slots per env, {batch['sweeps_mean']:.2f} sweeps used on "
                f"average, {batch['envs_at_sweep_cap']} envs at the cap of {cfg.vel_iters}")
    world.close()
    out = {
        "value": E * 1e3 / wall_ms, "ms_per_step": wall_ms, "steps": steps, "warmup": warmup,
        "config": {"workload": f"{cfg.name}: {nl} links, {nv} DoF, {nc} contact " + ("slots of up to four points" if index == 6 else "spheres") + f", {E} envs, dt {cfg.dt:.6f}, "
                               f"{cfg.vel_iters} block-descent sweeps{live}" + (f"; {cfg.note}" if cfg.note else "")
                               + ("" if law == "native" else f"; MuJoCo contact law, {law} cone"),
                   "config_index": index, "envs": E,
                   "execution": mode, "event_ms_per_step": event_ms,
                   "each_step_from": "seeded batch (checkpoint restore inside the timed region)", **batch},
        "roofline": {"bound": "hbm", "kernel": kernel, "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": traffic,
                     "algorithmic_bytes_per_launch": kernel_bytes * E, "kernel_ms": kernel_ms,
                     "frac_survey": survey_gbps / HBM_PEAK_GBPS, "survey_bytes_per_launch": b_alg * E,
                     "solver_width": solver_width, "blocks_per_cu": blocks_per_cu, "waves_per_simd": blocks_per_cu / 4.0,
                     "profiled": profiled},
        "roofline_step": {"algorithmic_bytes_per_env_step": b_alg, "state_io_bytes_per_env_step": tier_a,
                          "achieved": step_gbps, "unit": "GB/s", "frac": step_gbps / HBM_PEAK_GBPS},
        "per_op_ms": {k: round(v, 4) for k, v in per_op.items() if v >= 0.001},
    }
    if cpu_budget_s > 0:
        out["cpu_baseline"] = cpu_baseline(nk, cfg, desc, cpu_budget_s)
    return out


# the other published configurations, timed in the same run with a short protocol: (config, envs, steps, warm-up)
OTHER_CONFIGS = [(1, 64, 200, 50), (2, 4096, 200, 50), (4, 1024, 200, 50), (4, 16384, 100, 30), (4, 65536, 40, 10), (5, 8192, 40, 10)]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--config", type=int, default=3)
    ap.add_argument("--envs", type=int, default=0)
    ap.add_argument("--mode", choices=("eager", "graph"), default="graph")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--contact-law", choices=("native", "elliptic", "pyramidal"), default="native",
                    help="with --only: the configuration's contacts under the MuJoCo law with this cone instead of the native law")
    ap.add_argument("--only", action="store_true", help="the named configuration alone, without the short runs of the others")
    ap.add_argument("--seeded-only", action="store_true",
                    help="kept for the profile commands: every launch of a run is a step from the seeded batch")
    ap.add_argument("--scene", default="", help="a scene file instead of a benchmark configuration: its robot left to itself (see scene_run)")
    ap.add_argument("--native-laws", action="store_true",
                    help="with --scene: the file's contacts and joint rows under the native laws (an MJCF file's are MuJoCo's by default)")
    ap.add_argument("--settle", type=int, default=600)
    ap.add_argument("--base-height", type=float, default=0.0, help="with --scene: height of the root link at the start, 0 keeps the file's")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path runs on one GPU (one wavefront per environment, no cross-device state); "
                 "--gpus must be 1")

    nk = entry.load_package()
    if args.scene:
        scene_run(nk, args)
        return
    device = nk.Device(0)
    if args.contact_law != "native" and not args.only:
        sys.exit("bench.py: --contact-law goes with --only (the published configurations use the native law)")
    head = measure(nk, device, args.config, args.envs, args.steps, args.warmup, args.mode, 0.0 if args.no_cpu_baseline else 12.0,
                   args.contact_law)
    result = {
        "metric": "env-steps/sec", "value": head["value"], "unit": "env-steps/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": head["ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": head["config"], "roofline": head["roofline"], "roofline_step": head["roofline_step"],
        "per_op_ms": head["per_op_ms"], "copy_ceiling_gbps": device.copy_bandwidth(1 << 28, 10),
        "tolerances": {"stated": 1e-4, "per_env": True,
                       "relaxed": "per-row lambda on the humanoid and qdd/velocity/lambda on the rope are held to max(1e-4, 4 x the "
                                  "oracle's own one-ulp input sensitivity): coplanar spheres on one rigid foot split the foot's impulse "
                                  "indeterminately (J^T lambda and velocities meet 1e-4); the rope's Newton block has cond ~1e6",
                       "against_double_precision": "largest distance per environment to the oracle built in double, device / single-precision "
                                                   "oracle, measured by tests/test_gpu_parity.py on 512 (rope: 64) environments: humanoid lambda "
                                                   "9.3e-4 / 6.2e-4, velocity 2.4e-4 / 2.4e-4, medians 1e-6; rope lambda 1.2e-3 / 1.7e-3, velocity "
                                                   "1.7e-4 / 2.0e-4, qdd 5.3e-4 / 4.6e-4; the test bounds the device's median, 95th percentile and "
                                                   "maximum by max(1e-4, 2 x the oracle's)"},
    }
    if "cpu_baseline" in head:
        result["cpu_baseline"] = head["cpu_baseline"]
    if not args.only and args.config == 3 and not args.envs:
        others = []
        for index, envs, steps, warmup in OTHER_CONFIGS:
            entry_ = measure(nk, device, index, envs, steps, warmup, args.mode, 0.0 if args.no_cpu_baseline else 2.5)
            entry_["unit"] = "env-steps/s"
            others.append(entry_)
        result["other_configs"] = others
    device.close()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
