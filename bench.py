#!/usr/bin/env python3
"""Benchmark of the batch=1 MoE decode hot path on one MI355X.

Workload (the 48-layer stack of the full-scale layer, mode A): a stack of 48 MoE layers (hidden 2048, 512 experts,
top-10, ffn 512, IQ3_S gate/up, Q8_0 down, Q8_0 shared expert gated by sigmoid(w.x), f32 router),
all 24,576 experts resident in HBM, one token per step.  Per layer the router runs and its weights
are used; the expert ids are replayed from a seeded Zipf(1.1) trace, as the workload prescribes.
One "step" = one token through the 48 layers.  Weights are synthetic (random GGUF block bytes with
the prescribed scale distributions) and are generated on the device before the timed region.

Prints ONE JSON line (see the keys at the bottom).  `value` is tokens/s with everything resident
in HBM; `roofline` prices the dominant kernel against the 8 TB/s HBM peak; `cpu_baseline` times the
reference's CPU MoE path (oracle/_ref when built, else the C port) on a bounded sample; `mode_b` is a
bounded run of the same stack with its routed experts in pinned host memory behind the slot pool.
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

HBM_PEAK_GBS = 8000.0
STACK_FLAGS = int(os.environ.get("WD_BENCH_FLAGS", "0"))   # experiments only (e.g. 4 = staged dispatches)
CHAIN_FLAGS = int(os.environ.get("WD_BENCH_CHAIN_FLAGS", "0"))   # experiments only (0x80 = launch floor)
TOKEN_MIX = float(os.environ.get("WD_BENCH_TOKEN_MIX", "0.6"))   # tokens mode: share of the common direction in every token
RESIDUAL_SCALE = 2.0 ** -12   # glue between layers: x += scale * layer(x), keeps the chain finite


def note(msg):
    print("[bench %.1fs] %s" % (time.perf_counter() - T0, msg), file=sys.stderr, flush=True)


T0 = time.perf_counter()


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--layers", type=int, default=48)
    ap.add_argument("--experts", type=int, default=512)
    ap.add_argument("--routing", choices=["zipf", "router"], default="zipf",
                    help="zipf: ids replayed from the Zipf(1.1) trace; router: ids chosen by the router itself")
    ap.add_argument("--mode", choices=["resident", "lru", "q4-sweep", "q8-sweep", "q8-batch", "q6k-head", "hc", "tokens", "c0", "model-layer"], default="resident",
                    help="resident: C3 mode A, every expert in HBM; lru: C3 mode B, experts in pinned host memory "
                         "behind an LRU slot pool of --cache-gib in HBM; q4-sweep: the dense Q4_0 GEMV shapes; "
                         "tokens: the 4-token speculative-verify pass over the same layers; c0: the 64-expert top-8 "
                         "all-Q8_0 layer (secondary workloads, own JSON lines)")
    ap.add_argument("--tokens", type=int, default=4, help="tokens mode: tokens per pass (<= 8)")
    ap.add_argument("--cache-gib", type=float, default=32.0)
    ap.add_argument("--fill", choices=["kernel", "memcpy"], default="kernel",
                    help="lru mode: fill misses with the copy kernel that reads pinned host memory, or with hipMemcpyAsync")
    ap.add_argument("--source", choices=["pinned", "file", "mapping"], default="pinned",
                    help="lru mode: where the routed experts live - pinned host memory; a GGUF file written to --file-dir, "
                         "misses read with pread into the cache's pinned ring; the same file as a plain (pageable) mapping")
    ap.add_argument("--host-layout", choices=["tensors", "packed"], default="tensors",
                    help="lru mode with --source pinned: the host copy as three tensors per layer (as in a model file), or packed "
                         "per expert - gate, up and down of an expert back to back, one slot apart - so that a miss is one "
                         "contiguous piece")
    ap.add_argument("--file-dir", default="/tmp", help="lru mode with --source file/mapping: directory of the model file")
    ap.add_argument("--pread-threads", type=int, default=4)
    ap.add_argument("--lru-driver", choices=["trace", "router"], default="trace",
                    help="lru mode: the host knows the routing trace and acquires a token's experts ahead (default), or every layer's "
                         "selection comes back from the device before its experts are acquired (what a decode loop without a "
                         "predictor does)")
    ap.add_argument("--read-ahead", type=int, default=0,
                    help="lru mode with --lru-driver router and --source file: layers of read-ahead (the previous token's experts are "
                         "read from the file into a pinned ring while the layers compute)")
    ap.add_argument("--cache-warm-tokens", type=int, default=256,
                    help="lru mode: tokens run before the warm-up steps so that the slot pool is in steady state")
    ap.add_argument("--cache-timing", action="store_true",
                    help="lru mode: switch on the cache's device-side timings (the copy stream's waits and fills, in the monitor "
                         "object); the events they need cost about 4 % of the rate")
    ap.add_argument("--graph", choices=["auto", "on", "off"], default="auto",
                    help="replay the step from a captured HIP graph or launch it eagerly; auto: eagerly when the step is one "
                         "launch (the resident stack: a graph of one kernel costs more than the launch it saves), a graph for "
                         "the dispatches per layer")
    ap.add_argument("--no-graph", action="store_true", help="the same as --graph off")
    ap.add_argument("--path", choices=["resident", "per-layer"], default="resident",
                    help="resident mode: the stack as ONE launch of resident workgroups (default), or two dispatches per layer")
    ap.add_argument("--repeats", type=int, default=5, help="further repeats of the timed region, for the spread in the JSON line")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-mode-b", action="store_true",
                    help="resident mode: leave out the bounded run of the same stack with its experts behind the slot pool")
    ap.add_argument("--site-profile", type=int, default=0, metavar="TOKENS",
                    help="resident mode: afterwards run TOKENS eager steps with the library's site profiler on (device, host and "
                         "gap time per bracketed site and token), print its report and add it to the JSON line")
    ap.add_argument("--cpu-seconds", type=float, default=12.0,
                    help="wall-clock seconds of CPU layer passes to accumulate for cpu_baseline (all host threads busy)")
    ap.add_argument("--check", action="store_true", help="verify one layer pass against the CPU oracle first")
    return ap.parse_args()


def offload_layer(capi, torch, synth, t, d, packed):
    """Moves one layer's routed tensors (device tensors in `t`, pointers in descriptor `d`) to pinned host memory and
    drops their device copies; returns the three host pointers.  `packed`: one buffer, gate, up and down of an expert
    back to back, experts one slot apart."""
    H, F, n_experts = 2048, 512, d.n_experts
    gbytes, dbytes = F * synth.row_bytes(synth.IQ3_S, H), H * synth.row_bytes(synth.Q8_0, F)
    if packed:
        slot = torch.cat([t["gate"].view(n_experts, gbytes), t["up"].view(n_experts, gbytes),
                          t["down"].view(n_experts, dbytes)], dim=1).contiguous()
        h = C.c_void_p()
        capi.call("wd_malloc_host", C.byref(h), slot.numel())
        capi.call("wd_memcpy_d2h", h, C.c_void_p(slot.data_ptr()), slot.numel(), None)
        del slot
        host = [h, C.c_void_p(h.value + gbytes), C.c_void_p(h.value + 2 * gbytes)]
    else:
        host = []
        for name in ("gate", "up", "down"):
            h = C.c_void_p()      # exact-size pinned buffer (torch's pinned allocator rounds sizes up to 2^n)
            capi.call("wd_malloc_host", C.byref(h), t[name].numel())
            capi.call("wd_memcpy_d2h", h, C.c_void_p(t[name].data_ptr()), t[name].numel(), None)
            host.append(h)
    for name in ("gate", "up", "down"):
        t[name] = None
        setattr(d, name, None)
    return host


def build_stack(torch, synth, capi, n_layers, n_experts, seed, offload=False, packed=False):
    """Random GGUF-layout weights for n_layers C2 layers, generated on the device.  With `offload` the routed
    tensors are moved to pinned host memory (returned per layer) and their device copies dropped; `packed` lays
    them out per expert (gate, up, down of expert e back to back, experts one slot apart) in ONE buffer per layer and
    returns that buffer's three starting points."""
    H, F, k = 2048, 512, 10
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    rb_iq3, rb_q8h, rb_q8f = synth.row_bytes(synth.IQ3_S, H), synth.row_bytes(synth.Q8_0, H), synth.row_bytes(synth.Q8_0, F)

    def iq3(rows):
        t = torch.randint(0, 256, (rows * rb_iq3,), dtype=torch.uint8, device="cuda", generator=g)
        d = (torch.randn(rows * (H // 256), device="cuda", generator=g).abs() * 0.01).half()
        t.view(-1, 110)[:, 0:2] = d.view(torch.uint8).view(-1, 2)
        return t

    def q8(rows, cols):
        nb = rows * (cols // 32)
        t = torch.randint(-127, 128, (nb * 34,), dtype=torch.int8, device="cuda", generator=g).view(torch.uint8)
        d = (torch.randn(nb, device="cuda", generator=g).abs() * (0.02 / 127.0)).half()
        t.view(-1, 34)[:, 0:2] = d.view(torch.uint8).view(-1, 2)
        return t

    layers, keep, pinned = (capi.MoeLayer * n_layers)(), [], []
    for l in range(n_layers):
        t = dict(router=torch.randn(n_experts, H, device="cuda", generator=g) * (1.0 / np.sqrt(H)),
                 gate=iq3(n_experts * F), up=iq3(n_experts * F), down=q8(n_experts * H, F),
                 shared_gate_inp=torch.randn(H, device="cuda", generator=g) * 0.02,
                 shared_gate=q8(F, H), shared_up=q8(F, H), shared_down=q8(H, F))
        keep.append(t)
        d = layers[l]
        d.hidden, d.expert_ffn, d.n_experts, d.top_k, d.expert_scale = H, F, n_experts, k, 1.0
        d.gate_type = d.up_type = synth.IQ3_S
        d.down_type = synth.Q8_0
        for name, tensor in t.items():
            setattr(d, name, tensor.data_ptr())
        d.gate_stride = d.up_stride = F * rb_iq3
        d.down_stride = H * rb_q8f
        if offload:
            pinned.append(offload_layer(capi, torch, synth, t, d, packed))
    return (layers, keep, pinned) if offload else (layers, keep)


def layer_dict(torch, synth, t, n_experts):
    """Host copy of one device layer in the dict form the CPU checker takes."""
    L = dict(hidden=2048, expert_ffn=512, n_experts=n_experts, top_k=10, w_scale=1.0, gate_type=synth.IQ3_S,
             up_type=synth.IQ3_S, down_type=synth.Q8_0, shared_type=synth.Q8_0)
    for name, tensor in t.items():
        a = tensor.cpu().numpy()
        L[name] = a.reshape(n_experts, -1) if name in ("gate", "up", "down") else a
    return L


CPU_LAYERS, CPU_EXPERTS = 4, 512      # 4 x 1.03 GB of weights: far beyond any last-level cache


def cpu_weights(folder):
    """Writes the cpu_baseline leg's weights as .npy files that its children map: 128 experts generated like the GPU
    workload's, every layer made of those blocks four times over in an order of its own (1.03 GB of distinct memory
    per layer), with small tensors of its own."""
    from warpdecode_amd import synth
    made = 128
    base = synth.make_c2(layer=0, n_experts=made)
    rng = synth.rng_for(synth.BASE_SEED, 9003)
    for l in range(CPU_LAYERS):
        order = rng.permutation(np.tile(np.arange(made), CPU_EXPERTS // made))
        small = base if l == 0 else synth.make_c2(layer=l, n_experts=8)
        for name, a in base.items():
            if not isinstance(a, np.ndarray):
                continue
            if name in ("gate", "up", "down", "router"):
                a = a.reshape(made, -1)[order].reshape((CPU_EXPERTS,) + a.shape[1:])
            elif l > 0:
                a = small[name]
            np.save(os.path.join(folder, "%d.%s.npy" % (l, name)), a)


def cpu_child(seconds, threads, kind, folder):
    """Child process of the cpu_baseline leg: no GPU.  Times layer passes of the headline workload's shape (512
    experts per layer, ids Zipf(1.1) over a permutation of its own per layer, 4 layers' weights taken in turn) in the
    C port of the layer, or in the reference CPU MoE path (its run_layer + thread pool for the routed experts, its
    Q8_0 row kernels for the shared expert; router through the C port), and prints one progress line per pass."""
    from oracle import pyoracle
    from warpdecode_amd import synth
    proto = synth.make_c2(layer=0, n_experts=8)
    layers = []
    for l in range(CPU_LAYERS):
        L = {k: v for k, v in proto.items() if not isinstance(v, np.ndarray)}
        L["n_experts"] = CPU_EXPERTS
        for name, a in proto.items():
            if isinstance(a, np.ndarray):
                L[name] = np.load(os.path.join(folder, "%d.%s.npy" % (l, name)), mmap_mode="r")
        layers.append(L)
    rng = synth.rng_for(synth.BASE_SEED, 9002)
    perms = [rng.permutation(CPU_EXPERTS) for _ in range(CPU_LAYERS)]
    x = synth.rms_normed(rng, 2048)
    for L in layers:                      # fault the mappings in before the clock starts
        for name in ("gate", "up", "down", "router"):
            np.add.reduce(L[name].reshape(-1)[::4096], dtype=np.uint64 if L[name].dtype == np.uint8 else None)
    print("READY", flush=True)
    passes, t0 = 0, time.perf_counter()
    while True:
        l = passes % CPU_LAYERS
        L = layers[l]
        ids = synth.zipf_ids(rng, CPU_EXPERTS, 10, 1.1, perms[l])
        logits = pyoracle.router_logits(L["router"], x)
        _, wts = pyoracle.route(logits, 10)
        if kind == "reference":
            out = pyoracle.ref_run_layer(L, x, ids, wts, threads=threads)
            sh = pyoracle.ref_q8_0_chain(L["shared_gate"], L["shared_up"], L["shared_down"], 2048, 512, x)
            gate = pyoracle.sigmoid_ggml(pyoracle.dot_f32(L["shared_gate_inp"], x))
            out = (out + (sh * gate).astype(np.float32)).astype(np.float32)
        else:
            out, _ = pyoracle.moe_layer(L, x, ids=ids, weights=wts, threads=threads)
        passes += 1
        dt = time.perf_counter() - t0
        print("P %d %.6f" % (passes, dt), flush=True)
        if dt >= seconds and passes >= 8:
            break


def cpu_leg(kind, seconds, threads, folder, max_children):
    """Runs cpu_child as fresh child processes until `seconds` of timed passes have accumulated (or the children run
    out).  A child that prints nothing for 2.5 s after its first pass has stalled (the reference's fork-join pool can
    dead-lock when a late worker picks up a task of the next parallel_for): it is killed, the passes it completed
    count, and a fresh child continues.  Returns (passes, seconds, stalled children)."""
    import subprocess
    import threading
    tot_passes, tot_time, stalls = 0, 0.0, 0
    for _ in range(max_children):
        remaining = seconds - tot_time
        if remaining <= 0.5:
            break
        proc = subprocess.Popen([sys.executable, os.path.abspath(__file__), "--cpu-child", str(remaining), str(threads), kind, folder],
                                stdout=subprocess.PIPE, stderr=subprocess.DEVNULL, text=True)
        last = [0, 0.0, time.perf_counter()]

        def reader():
            for line in proc.stdout:
                f = line.split()
                if f and f[0] == "P":
                    last[0], last[1] = int(f[1]), float(f[2])
                last[2] = time.perf_counter()

        th = threading.Thread(target=reader, daemon=True)
        th.start()
        while proc.poll() is None:
            time.sleep(0.25)
            # a pass takes milliseconds; only the start-up (mapping 4 GB of weights) is slow
            if time.perf_counter() - last[2] > (90.0 if last[0] == 0 else 2.5):
                stalls += 1
                proc.kill()
                break
        proc.wait()
        th.join(timeout=5)
        tot_passes += last[0]
        tot_time += last[1]
    return tot_passes, tot_time, stalls


def cpu_baseline(seconds):
    """The layer pass on the host cores, on the headline workload's shape.  `value` is the reference's own CPU MoE path
    (kind "reference") when its build is present, with the number of its children that stalled beside it; the C port of
    the layer (one child, no restarts) is reported under "port", and is `value` (kind "port") where the reference
    build is absent.  ms/layer is converted to tokens/s of a 48-layer stack."""
    import shutil
    import tempfile
    from oracle import pyoracle
    cpus = len(os.sched_getaffinity(0))
    threads = max(1, min(cpus, 16))
    folder = tempfile.mkdtemp(prefix="wd_cpu_", dir="/dev/shm" if os.path.isdir("/dev/shm") else None)
    workload = ("layer passes of the headline shape (hidden 2048, ffn 512, top-10 of %d experts + shared expert, ids "
                "Zipf(1.1) over a per-layer permutation, %d layers = %.1f GB of weights taken in turn)"
                % (CPU_EXPERTS, CPU_LAYERS, CPU_LAYERS * 1.039))

    def leg(kind, children):
        passes, secs, stalls = cpu_leg(kind, seconds, threads, folder, children)
        note("cpu baseline (%s): %d passes in %.1f s, %d stalled children" % (kind, passes, secs, stalls))
        if passes < 8:
            return dict(value=None, unit="tok/s", cores=threads, kind=kind, stalled_children=stalls,
                        sample="fewer than 8 CPU passes completed")
        per_layer = secs / passes
        return dict(value=round(1.0 / (per_layer * 48), 3), unit="tok/s", cores=threads, kind=kind, stalled_children=stalls,
                    passes=passes, seconds=round(secs, 2), ms_per_layer=round(per_layer * 1e3, 3),
                    sample="%d %s in %.1f s = %.2f ms/layer, x48 layers per token; %d threads on %d host cores"
                           % (passes, workload, secs, per_layer * 1e3, threads, cpus))
    try:
        note("cpu baseline: writing %d layers of weights to %s" % (CPU_LAYERS, folder))
        cpu_weights(folder)
        port = leg("port", 1)
        port["sample"] += "; C restatement of the layer, one child process, no restarts"
        if pyoracle.ref() is None:
            return port
        out = leg("reference", 12)
        out["sample"] += ("; the reference's own CPU MoE path built from its sources; a child whose thread pool dead-locked "
                          "was killed and replaced by a fresh one (stalled_children), only completed passes count")
        out["port"] = port
        return out
    finally:
        shutil.rmtree(folder, ignore_errors=True)


def recorded_traffic(kernel):
    """HBM bytes per launch of `kernel` as recorded from hardware-counter runs of this command (the file
    says how they were taken and scaled); None when no record exists for this kernel."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic_c3_mode_a.txt")
    try:
        for line in open(path):
            f = line.split()
            if len(f) >= 3 and f[0] == "traffic_bytes" and f[1] == kernel:
                return int(f[2])
    except OSError:
        pass
    return None


def bench_lru(args, torch, capi, synth, stack=None):
    """C3 mode B: the routed experts live in pinned host memory; an LRU pool of --cache-gib in HBM holds the
    recently used ones.  The routing trace is known to the host, so the fills of layer l+1 are queued while
    layer l computes.  Eager launches (the cache decides per token what to copy).  Returns the JSON object.
    `stack`: (layers, keep) of a stack already on the device, whose routed tensors are then moved to pinned host
    memory in place (--source pinned only)."""
    H, F, k, E, NL = 2048, 512, 10, args.experts, args.layers
    gb, db = F * synth.row_bytes(synth.IQ3_S, H), H * synth.row_bytes(synth.Q8_0, F)
    slot_bytes = 2 * gb + db
    cache = C.c_void_p()
    model_file = None
    if args.source == "pinned":
        note("generating %d layers x %d experts, routed tensors to pinned host memory" % (NL, E))
        packed = args.host_layout == "packed"
        if stack is None:
            layers, keep, pinned = build_stack(torch, synth, capi, NL, E, synth.BASE_SEED, offload=True, packed=packed)
        else:
            layers, keep = stack
            pinned = [offload_layer(capi, torch, synth, keep[l], layers[l], packed) for l in range(NL)]
            torch.cuda.empty_cache()
        torch.cuda.synchronize()
        capi.call("wd_expert_cache_create", C.byref(cache), int(args.cache_gib * (1 << 30)), gb, gb, db, NL, E, 0)
        capi.call("wd_expert_cache_set_copy_kernel", cache, 1 if args.fill == "kernel" else 0)
        for l in range(NL):
            if packed:
                capi.call("wd_expert_cache_register_layer_strided", cache, l, *pinned[l], slot_bytes, slot_bytes, slot_bytes)
            else:
                capi.call("wd_expert_cache_register_layer", cache, l, *pinned[l])
    else:
        # the routed tensors go into a GGUF file (names of the model files), are dropped from the device, and come back
        # through the library's reader: the cache's host sources are pointers into its mapping
        from warpdecode_amd import ggufio
        layers, keep = build_stack(torch, synth, capi, NL, E, synth.BASE_SEED)
        path = os.path.join(args.file_dir, "wd_bench_%d_%dx%d.gguf" % (os.getpid(), NL, E))
        note("writing %d layers x %d experts (%.1f GB) to %s" % (NL, E, NL * E * slot_bytes / 1e9, path))
        tensors = []
        for l in range(NL):
            for name, dims, ttype in (("gate", [H, F, E], synth.IQ3_S), ("up", [H, F, E], synth.IQ3_S), ("down", [F, H, E], synth.Q8_0)):
                tensors.append(("blk.%d.ffn_%s_exps.weight" % (l, name), dims, ttype, keep[l][name].cpu().numpy()))
                keep[l][name] = None
                setattr(layers[l], name, None)
        torch.cuda.empty_cache()
        ggufio.write_gguf(path, tensors, [("general.architecture", ggufio.STRING, "qwen38")])
        del tensors
        model_file = ggufio.GgufFile(path)
        os.unlink(path)     # the open mapping and descriptor keep the file alive; nothing is left behind
        capi.call("wd_expert_cache_create", C.byref(cache), int(args.cache_gib * (1 << 30)), gb, gb, db, NL, E, 0)
        if args.source == "file":
            capi.call("wd_expert_cache_attach_file", cache, C.c_void_p(model_file.map_base), model_file.map_bytes, model_file.fd,
                      args.pread_threads)
        for l in range(NL):
            ptrs = [C.c_void_p(model_file.tensors["blk.%d.ffn_%s_exps.weight" % (l, n)]["ptr"]) for n in ("gate", "up", "down")]
            capi.call("wd_expert_cache_register_layer", cache, l, *ptrs)
    st_slots = int(args.cache_gib * (1 << 30)) // slot_bytes
    for policy, slots in ((0, st_slots // 2), (0, 2 * st_slots), (1, st_slots)):   # counterfactual pools, same accesses
        capi.call("wd_expert_cache_add_shadow", cache, policy, slots)
    if args.cache_timing:
        capi.call("wd_expert_cache_set_timing", cache, 1)
    scratch = C.c_void_p()
    capi.call("wd_moe_scratch_create", C.byref(scratch), H, F, E, k)
    st0 = capi.CacheStats()
    capi.call("wd_expert_cache_get_stats", cache, C.byref(st0))
    note("pool: %d slots of %d B (%.1f GiB) for %d (layer, expert) pairs; host side (%s) %.1f GB"
         % (st0.slots, slot_bytes, st0.slots * slot_bytes / 2 ** 30, NL * E, args.source, NL * E * slot_bytes / 1e9))

    total = args.cache_warm_tokens + args.warmup + args.steps
    rng = synth.rng_for(synth.BASE_SEED, 9001)
    perms = [rng.permutation(E) for _ in range(NL)]
    trace = np.stack([np.stack([synth.zipf_ids(rng, E, k, 1.1, perms[l]) for l in range(NL)])
                      for _ in range(total)]).astype(np.int32)
    xs = np.stack([synth.rms_normed(rng, H) for _ in range(64)])
    d_trace_all, d_xs = torch.from_numpy(trace).cuda(), torch.from_numpy(xs).cuda()
    d_x = torch.zeros(H, dtype=torch.float32, device="cuda")
    d_out = torch.zeros(H, dtype=torch.float32, device="cuda")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)

    if args.read_ahead:
        capi.call("wd_expert_cache_set_read_ahead", cache, args.read_ahead, 0)

    lru_flags = 0x200 if args.path == "per-layer" else 0     # WD_MOE_PER_LAYER

    def step(i):
        d_x.copy_(d_xs[i % 64], non_blocking=True)
        if args.lru_driver == "router":   # the router's own selection, layer by layer through the host
            capi.call("wd_moe_stack_cached_f32", layers, NL, cache, C.c_void_p(d_x.data_ptr()), C.c_void_p(d_out.data_ptr()),
                      scratch, None, None, RESIDUAL_SCALE, 0, stream)
            return
        capi.call("wd_moe_stack_cached_f32", layers, NL, cache, C.c_void_p(d_x.data_ptr()), C.c_void_p(d_out.data_ptr()),
                  scratch, trace[i].ctypes.data_as(C.c_void_p), C.c_void_p(d_trace_all[i].data_ptr()), RESIDUAL_SCALE, lru_flags, stream)

    def stats():
        st = capi.CacheStats()
        capi.call("wd_expert_cache_get_stats", cache, C.byref(st))
        return st

    t0 = time.perf_counter()
    for i in range(args.cache_warm_tokens):
        step(i)
    torch.cuda.synchronize()
    sw = stats()
    note("cache warm-up: %d tokens in %.2f s, %d resident, hit rate so far %.3f"
         % (args.cache_warm_tokens, time.perf_counter() - t0, sw.resident, sw.hits / max(1, sw.accesses)))
    base = args.cache_warm_tokens
    for i in range(args.warmup):
        step(base + i)
    torch.cuda.synchronize()
    s0 = stats()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for i in range(args.steps):
        step(base + args.warmup + i)
    ev1.record()
    host_ms = (time.perf_counter() - t0) * 1e3 / args.steps      # the host's share: queueing a token, nothing awaited
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    s1 = stats()
    ms_per_step = ev0.elapsed_time(ev1) / args.steps
    acc, hits, miss = s1.accesses - s0.accesses, s1.hits - s0.hits, s1.misses - s0.misses
    moved = s1.bytes_copied - s0.bytes_copied
    lib = capi.load()
    need = lib.wd_expert_cache_dump_json(cache, None, 0)
    buf = C.create_string_buffer(need + 1)
    lib.wd_expert_cache_dump_json(cache, buf, need + 1)
    monitor = json.loads(buf.value.decode())
    for key in ("layer_access", "layer_misses"):
        monitor.pop(key, None)
    bytes_per_step = 27697152 * NL if E == 512 else None
    whole = bytes_per_step / (ms_per_step * 1e-3) / 1e9 if bytes_per_step else None
    out = {
        "metric": "MoE layer batch=1 decode: synthetic 48-layer tok/s (achieved HBM GB/s in roofline)",
        "value": round(1000.0 / ms_per_step, 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 dot products (IQ3_S/Q8_0 weights x Q8_K/Q8_0 activations), f32 accumulate",
        "data": "synthetic",
        "config": {"workload": "C3 mode B: %d-layer stack of the 512-expert top-10 IQ3_S/Q8_0 MoE layer, batch=1, routed "
                               "experts in pinned host memory behind a %.0f GiB LRU slot pool in HBM, Zipf(1.1) trace" % (NL, args.cache_gib),
                   "layers": NL, "experts": E, "top_k": k, "routing": "zipf" if args.lru_driver == "trace" else "router", "launch": "eager",
                   "path": ("one resident launch per token, fills land while it runs" if monitor.get("tokens_in_one_launch", 0) >= total
                            else "dispatches per layer"),
                   "source": args.source, "driver": args.lru_driver, "read_ahead": args.read_ahead,
                   "slots": int(s1.slots), "slot_bytes": int(slot_bytes), "cache_warm_tokens": args.cache_warm_tokens,
                   "hit_rate": round(hits / max(1, acc), 4), "misses_per_token": round(miss / args.steps, 2),
                   "host_link_bytes_per_token": int(moved / args.steps),
                   "host_link_GBps": round(moved / (ms_per_step * 1e-3 * args.steps) / 1e9, 2),
                   "host_ms_per_step": round(host_ms, 4),
                   "wall_s": round(wall, 3), "finite": bool(torch.isfinite(d_x).all().item()),
                   "monitor_whole_run": monitor},
        "roofline": {"bound": "hbm", "achieved": round(whole, 1) if whole else None, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(whole / HBM_PEAK_GBS, 4) if whole else None, "traffic": None,
                     "kernel": "whole step (kernel bytes only; the host-link bytes are in config)"},
    }
    torch.cuda.synchronize()
    capi.call("wd_moe_scratch_destroy", scratch)
    capi.call("wd_expert_cache_destroy", cache)
    if args.source == "pinned":
        for host in pinned:
            for h in (host[:1] if packed else host):
                capi.call("wd_free_host", h)
    return out


def graph_period_us(torch, launch, launches, reps):
    """Average period of one launch of `launch(i)`, i in [0, launches), captured once and replayed `reps` times."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch(0)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for i in range(launches):
            launch(i)
    for _ in range(max(2, reps // 4)):
        graph.replay()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / (reps * launches)


def bench_q4_sweep(args, torch, capi, synth):
    """Dense Q4_0 x Q8_0 GEMV at batch=1 over the Llama-3.2-1B shapes (the dense sweep workload).  Every launch
    of a chain reads another copy of the matrix, with enough copies (>= 1.5 GB) that nothing is served from the
    256 MB last-level cache; the period is taken over a captured chain, so it includes the launch gap."""
    shapes = [(2048, 2048), (8192, 2048), (2048, 8192), (128256, 2048)]     # rows x cols of the weight
    results = []
    for rows, cols in shapes:
        nbytes = rows * synth.row_bytes(synth.Q4_0, cols)
        copies = max(2, min(640, -(-int(1.5e9) // nbytes)))
        one = torch.from_numpy(synth.matrix(synth.Q4_0, synth.rng_for(synth.BASE_SEED, 77, rows, cols), min(rows, 8192), cols))
        one = one.reshape(-1).cuda()
        w = one.repeat(-(-rows // min(rows, 8192)))[:nbytes].repeat(copies).reshape(copies, nbytes)
        x = torch.from_numpy(synth.rng_for(synth.BASE_SEED, 78, cols).normal(0, 1, cols).astype(np.float32)).cuda()
        qs = torch.empty(cols, dtype=torch.int8, device="cuda")
        sc = torch.empty(cols // 32, dtype=torch.int16, device="cuda")
        y = torch.empty(rows, dtype=torch.float32, device="cuda")
        stream = lambda: C.c_void_p(torch.cuda.current_stream().cuda_stream)
        vp = lambda t: C.c_void_p(t.data_ptr())

        def gemv(i):
            capi.call("wd_gemv_q8_0_f32", synth.Q4_0, C.c_void_p(w[i % copies].data_ptr()), rows, cols, vp(qs), vp(sc), vp(y),
                      None, stream())

        def call(i):
            capi.call("wd_q8_0_quantize_f32", vp(x), cols, vp(qs), vp(sc), stream())
            gemv(i)

        call(0)
        torch.cuda.synchronize()
        launches = max(copies, 32)
        reps = max(3, int(1e11 // (nbytes * launches)))    # about 20 ms of streaming per timed region at full rate
        us = graph_period_us(torch, gemv, launches, reps)
        us_call = graph_period_us(torch, call, launches, reps)
        results.append(dict(rows=rows, cols=cols, bytes=nbytes, copies=copies, us_per_gemv=round(us, 3),
                            gbs=round(nbytes / us / 1e3, 1), frac=round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                            us_per_call_with_quantise=round(us_call, 3), finite=bool(torch.isfinite(y).all().item())))
        note("Q4_0 %dx%d: %.2f us, %.0f GB/s" % (rows, cols, us, nbytes / us / 1e3))
        del w, one
        torch.cuda.empty_cache()
    head = results[-1]
    print(json.dumps({
        "metric": "dense Q4_0 GEMV batch=1: achieved HBM GB/s (lm_head 128256x2048)", "value": head["gbs"], "unit": "GB/s",
        "n_gpus": 1, "higher_is_better": True, "vs_baseline": None, "dtype": "int8 dot products, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": "C1: Q4_0 x Q8_0 GEMV sweep, Llama-3.2-1B shapes, raw GGUF 18-byte blocks", "shapes": results},
        "roofline": dict(bound="hbm", achieved=head["gbs"], peak=HBM_PEAK_GBS, unit="GB/s", frac=head["frac"], traffic=None,
                         kernel="k_gemv_q4_stream", us_per_launch=head["us_per_gemv"], bytes_per_launch=head["bytes"])}))


def bench_model_layer(args, torch, capi, synth):
    """The layer at the model's own tensor types and shapes (hidden 2560, ffn 640, 512 experts, top-10, IQ2_S gate/up,
    IQ4_NL down, Q8_0 shared expert): `--layers` independent layers chained as in the headline workload,
    router-selected experts, one token per step."""
    H, F, k, E, NL = 2560, 640, 10, args.experts, min(args.layers, 16)
    g = torch.Generator(device="cuda")
    g.manual_seed(synth.BASE_SEED + 6)
    rb_g, rb_d = synth.row_bytes(synth.IQ2_S, H), synth.row_bytes(synth.IQ4_NL, F)
    rb_qh, rb_qf = synth.row_bytes(synth.Q8_0, H), synth.row_bytes(synth.Q8_0, F)

    def blocks(rows, cols, block_bytes, block_elems, scale):
        nb = rows * (cols // block_elems)
        t = torch.randint(0, 256, (nb * block_bytes,), dtype=torch.uint8, device="cuda", generator=g)
        d = (torch.randn(nb, device="cuda", generator=g).abs() * scale).half()
        t.view(-1, block_bytes)[:, 0:2] = d.view(torch.uint8).view(-1, 2)
        return t

    def q8(rows, cols):
        nb = rows * (cols // 32)
        t = torch.randint(-127, 128, (nb * 34,), dtype=torch.int8, device="cuda", generator=g).view(torch.uint8)
        d = (torch.randn(nb, device="cuda", generator=g).abs() * (0.02 / 127.0)).half()
        t.view(-1, 34)[:, 0:2] = d.view(torch.uint8).view(-1, 2)
        return t

    layers, keep = (capi.MoeLayer * NL)(), []
    for l in range(NL):
        t = dict(router=torch.randn(E, H, device="cuda", generator=g) * (1.0 / np.sqrt(H)),
                 gate=blocks(E * F, H, 82, 256, 0.0004), up=blocks(E * F, H, 82, 256, 0.0004), down=blocks(E * H, F, 18, 32, 0.0002),
                 shared_gate_inp=torch.randn(H, device="cuda", generator=g) * 0.02,
                 shared_gate=q8(F, H), shared_up=q8(F, H), shared_down=q8(H, F))
        keep.append(t)
        d = layers[l]
        d.hidden, d.expert_ffn, d.n_experts, d.top_k, d.expert_scale = H, F, E, k, 1.0
        d.gate_type = d.up_type = synth.IQ2_S
        d.down_type = synth.IQ4_NL
        for name, tensor in t.items():
            setattr(d, name, tensor.data_ptr())
        d.gate_stride = d.up_stride = F * rb_g
        d.down_stride = H * rb_d
    scratch = C.c_void_p()
    capi.call("wd_moe_scratch_create", C.byref(scratch), H, F, E, k)
    rng = synth.rng_for(synth.BASE_SEED, 9400)
    d_x = torch.from_numpy(synth.rms_normed(rng, H)).cuda()
    d_out = torch.zeros(H, dtype=torch.float32, device="cuda")

    def launch(_i):
        capi.call("wd_moe_stack_f32", layers, NL, C.c_void_p(d_x.data_ptr()), C.c_void_p(d_out.data_ptr()), scratch, None,
                  RESIDUAL_SCALE, 0, C.c_void_p(torch.cuda.current_stream().cuda_stream))

    us = graph_period_us(torch, launch, 1, 50) / NL
    finite, waits_ok = bool(torch.isfinite(d_x).all().item()), capi.load().wd_moe_scratch_status(scratch) == 0
    note("finite %s, |x| max %.3g, in-dispatch waits ok %s" % (finite, float(d_x.abs().max().item()), waits_ok))
    ok = finite and waits_ok
    nbytes = E * H * 4 + H * 4 + k * (2 * F * rb_g + H * rb_d) + 2 * F * rb_qh + H * rb_qf
    note("model-shape layer: %.2f us per layer, %.0f GB/s" % (us, nbytes / us / 1e3))
    print(json.dumps({
        "metric": "MoE layer batch=1 decode at the model's own types and shapes: us per layer", "value": round(us, 2), "unit": "us",
        "n_gpus": 1, "higher_is_better": False, "vs_baseline": None,
        "dtype": "int8 dot products (IQ2_S/IQ4_NL/Q8_0 weights x Q8_K/Q8_0 activations), f32 accumulate", "data": "synthetic",
        "config": {"workload": "%d chained layers of hidden 2560, %d experts, top-10, ffn 640, IQ2_S gate/up, IQ4_NL down, "
                               "Q8_0 shared expert, router-selected, batch=1, HIP-graph replay" % (NL, E),
                   "layers": NL, "bytes_per_layer": nbytes, "valid": ok},
        "roofline": dict(bound="hbm", achieved=round(nbytes / us / 1e3, 1), peak=HBM_PEAK_GBS, unit="GB/s",
                         frac=round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4), traffic=None,
                         kernel="whole layer (k_layer_ab<IQ2_S>, k_layer_c<IQ4_NL>)")}))


def bench_q8_sweep(args, torch, capi, synth):
    """Dense exact-order Q8_0 x Q8_0 GEMV at batch=1 (the projections around the MoE layer: hyper-connection mix, attention
    and recurrent blocks, src/qwen38_hc.cuh:1020-1049) over square, wide, tall and head-sized shapes.  Every launch of a
    chain reads another copy of the matrix (>= 1.5 GB of copies); the period is taken over a captured chain."""
    shapes = [(2048, 2048), (8192, 2048), (2048, 8192), (512, 8192), (8192, 512), (1024, 4096), (4096, 8192), (8192, 8192),
              (32768, 2048), (151936, 2048)]
    results = []
    for rows, cols in shapes:
        nbytes = rows * synth.row_bytes(synth.Q8_0, cols)
        copies = max(2, min(640, -(-int(1.5e9) // nbytes)))
        part = min(rows, 2048)
        one = torch.from_numpy(synth.matrix(synth.Q8_0, synth.rng_for(synth.BASE_SEED, 79, rows, cols), part, cols)).reshape(-1).cuda()
        w = one.repeat(-(-rows // part))[:nbytes].repeat(copies).reshape(copies, nbytes)
        x = torch.from_numpy(synth.rng_for(synth.BASE_SEED, 80, cols).normal(0, 1, cols).astype(np.float32)).cuda()
        qs = torch.empty(cols, dtype=torch.int8, device="cuda")
        sc = torch.empty(cols // 32, dtype=torch.int16, device="cuda")
        y = torch.empty(rows, dtype=torch.float32, device="cuda")
        stream = lambda: C.c_void_p(torch.cuda.current_stream().cuda_stream)
        vp = lambda t: C.c_void_p(t.data_ptr())
        capi.call("wd_q8_0_quantize_f32", vp(x), cols, vp(qs), vp(sc), stream())

        def gemv(i):
            capi.call("wd_gemv_q8_0_f32", synth.Q8_0, C.c_void_p(w[i % copies].data_ptr()), rows, cols, vp(qs), vp(sc), vp(y),
                      None, stream())

        gemv(0)
        torch.cuda.synchronize()
        launches = max(copies, 32)
        reps = max(3, int(1e11 // (nbytes * launches)))
        us = graph_period_us(torch, gemv, launches, reps)
        results.append(dict(rows=rows, cols=cols, bytes=nbytes, copies=copies, us_per_gemv=round(us, 3),
                            gbs=round(nbytes / us / 1e3, 1), frac=round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                            finite=bool(torch.isfinite(y).all().item())))
        note("Q8_0 %dx%d: %.2f us, %.0f GB/s" % (rows, cols, us, nbytes / us / 1e3))
        del w, one
        torch.cuda.empty_cache()
    head = results[-1]
    print(json.dumps({
        "metric": "dense Q8_0 GEMV batch=1: achieved HBM GB/s (151936x2048)", "value": head["gbs"], "unit": "GB/s",
        "n_gpus": 1, "higher_is_better": True, "vs_baseline": None, "dtype": "int8 dot products, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": "exact-order Q8_0 x Q8_0 GEMV sweep, raw GGUF 34-byte blocks", "shapes": results},
        "roofline": dict(bound="hbm", achieved=head["gbs"], peak=HBM_PEAK_GBS, unit="GB/s", frac=head["frac"], traffic=None,
                         kernel="k_gemv_q8_rows8", us_per_launch=head["us_per_gemv"], bytes_per_launch=head["bytes"])}))


def bench_q8_batch(args, torch, capi, synth):
    """The middle sizes of the exact-order Q8_0 GEMV as a block issues them: ten projections of one shape on one activation,
    as ten launches and as ONE launch (wd_gemv_q8_0_batch_f32).  Every launch of a chain reads another copy of its
    matrices (>= 1.5 GB of copies), the period is taken over a captured chain."""
    n_items = 10
    results = []
    for wtype, rows, cols in [(synth.Q8_0, 2048, 2048), (synth.Q8_0, 1024, 4096), (synth.Q8_0, 512, 8192), (synth.Q8_0, 512, 2048),
                              (synth.Q4_0, 2048, 2048), (synth.Q4_0, 512, 2048)]:
        tname = "Q8_0" if wtype == synth.Q8_0 else "Q4_0"
        nbytes = rows * synth.row_bytes(wtype, cols)
        sets = max(2, -(-int(1.5e9) // (nbytes * n_items)))
        one = torch.from_numpy(synth.matrix(wtype, synth.rng_for(synth.BASE_SEED, 83, rows, cols), rows, cols)).reshape(-1).cuda()
        w = one.repeat(sets * n_items).reshape(sets, n_items, nbytes)
        x = torch.from_numpy(synth.rng_for(synth.BASE_SEED, 84, cols).normal(0, 1, cols).astype(np.float32)).cuda()
        qs = torch.empty(cols, dtype=torch.int8, device="cuda")
        sc = torch.empty(cols // 32, dtype=torch.int16, device="cuda")
        y = torch.empty((n_items, rows), dtype=torch.float32, device="cuda")
        y1 = torch.empty((n_items, rows), dtype=torch.float32, device="cuda")
        stream = lambda: C.c_void_p(torch.cuda.current_stream().cuda_stream)
        vp = lambda t: C.c_void_p(t.data_ptr())
        capi.call("wd_q8_0_quantize_f32", vp(x), cols, vp(qs), vp(sc), stream())
        tables = []
        for s_ in range(sets):
            items = (capi.GemvItem * n_items)()
            for i in range(n_items):
                items[i].d_w, items[i].rows, items[i].d_act_qs, items[i].d_act_scales, items[i].d_out = (
                    w[s_, i].data_ptr(), rows, qs.data_ptr(), sc.data_ptr(), y[i].data_ptr())
            tables.append(items)

        def batched(j):
            capi.call("wd_gemv_q8_0_batch_f32", wtype, tables[j % sets], n_items, cols, stream())

        def single(j):
            for i in range(n_items):
                capi.call("wd_gemv_q8_0_f32", wtype, C.c_void_p(w[j % sets, i].data_ptr()), rows, cols, vp(qs), vp(sc), vp(y1[i]),
                          None, stream())

        batched(0)
        single(0)
        torch.cuda.synchronize()
        same = bool(torch.equal(y.view(torch.int32), y1.view(torch.int32)))
        launches = max(sets, 8)
        reps = max(3, int(1e11 // (nbytes * n_items * launches)))
        us_b = graph_period_us(torch, batched, launches, reps)
        us_s = graph_period_us(torch, single, launches, reps)
        results.append(dict(type=tname, rows=rows, cols=cols, items=n_items, bytes_per_item=nbytes, sets=sets, same_bits=same,
                            us_per_gemv_batched=round(us_b / n_items, 3), us_per_gemv_single=round(us_s / n_items, 3),
                            gbs_batched=round(nbytes * n_items / us_b / 1e3, 1), gbs_single=round(nbytes * n_items / us_s / 1e3, 1),
                            frac_batched=round(nbytes * n_items / us_b / 1e3 / HBM_PEAK_GBS, 4),
                            frac_single=round(nbytes * n_items / us_s / 1e3 / HBM_PEAK_GBS, 4)))
        note("%s %dx%d x %d: %.2f us per GEMV in one launch (%.0f GB/s), %.2f us one launch each (%.0f GB/s), same bits %s"
             % (tname, rows, cols, n_items, us_b / n_items, nbytes * n_items / us_b / 1e3, us_s / n_items, nbytes * n_items / us_s / 1e3, same))
        del w, one
        torch.cuda.empty_cache()
    head = results[0]
    print(json.dumps({
        "metric": "ten exact-order Q8_0 GEMVs 2048x2048 in one launch, batch=1: achieved HBM GB/s", "value": head["gbs_batched"],
        "unit": "GB/s", "n_gpus": 1, "higher_is_better": True, "vs_baseline": None, "dtype": "int8 dot products, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": "the middle sizes of the dense GEMVs (exact-order Q8_0, Q4_0) against Q8_0 activations, ten projections per "
                               "launch against ten launches",
                   "shapes": results, "valid": all(r["same_bits"] for r in results)},
        "roofline": dict(bound="hbm", achieved=head["gbs_batched"], peak=HBM_PEAK_GBS, unit="GB/s", frac=head["frac_batched"],
                         traffic=None, kernel="k_gemv_q8_rows8_split_batch", us_per_launch=round(head["us_per_gemv_batched"] * n_items, 3),
                         bytes_per_launch=head["bytes_per_item"] * n_items)}))
    if not all(r["same_bits"] for r in results):
        sys.exit(1)


def bench_q6k_head(args, torch, capi, synth):
    """The output head of the Qwen3 MoE models: Q6_K 151936 x 2048 against the Q8_K image of the F32 activation, once
    per decoded token.  Every launch of a chain reads another copy of the matrix (7 copies, 1.8 GB) so that nothing
    comes from the 256 MB last-level cache; the period is taken over a captured chain and includes the launch gap."""
    rows, cols = 151936, 2048
    nbytes = rows * synth.row_bytes(synth.Q6_K, cols)
    copies = 7
    part = torch.from_numpy(synth.matrix(synth.Q6_K, synth.rng_for(synth.BASE_SEED, 81, rows, cols), 4748, cols)).reshape(-1).cuda()
    w = part.repeat(rows // 4748)[:nbytes].repeat(copies).reshape(copies, nbytes)
    x = torch.from_numpy(synth.rms_normed(synth.rng_for(synth.BASE_SEED, 82, cols), cols)).cuda()
    qs = torch.empty(cols, dtype=torch.int8, device="cuda")
    sc = torch.empty(cols // 256, dtype=torch.float32, device="cuda")
    bs = torch.empty(cols // 16, dtype=torch.int16, device="cuda")
    y = torch.empty(rows, dtype=torch.float32, device="cuda")
    stream = lambda: C.c_void_p(torch.cuda.current_stream().cuda_stream)
    vp = lambda t: C.c_void_p(t.data_ptr())

    def gemv(i):
        capi.call("wd_gemv_q6_k_q8_k_f32", C.c_void_p(w[i % copies].data_ptr()), rows, cols, vp(qs), vp(sc), vp(bs), vp(y), None, stream())

    def call(i):
        capi.call("wd_q8_k_quantize_f32", vp(x), cols, vp(qs), vp(sc), vp(bs), stream())
        gemv(i)

    call(0)
    torch.cuda.synchronize()
    launches = 28
    reps = max(3, int(1e11 // (nbytes * launches)))
    us = graph_period_us(torch, gemv, launches, reps)
    us_call = graph_period_us(torch, call, launches, reps)
    gbs = nbytes / us / 1e3
    note("Q6_K head %dx%d: %.2f us, %.0f GB/s" % (rows, cols, us, gbs))
    print(json.dumps({
        "metric": "Q6_K x Q8_K output head batch=1: achieved HBM GB/s (151936x2048)", "value": round(gbs, 1), "unit": "GB/s",
        "n_gpus": 1, "higher_is_better": True, "vs_baseline": None, "dtype": "int8 dot products, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": "output head: Q6_K x Q8_K GEMV 151936x2048, raw GGUF 210-byte super-blocks", "bytes": nbytes,
                   "copies": copies, "us_per_call_with_quantise": round(us_call, 3), "finite": bool(torch.isfinite(y).all().item())},
        "roofline": dict(bound="hbm", achieved=round(gbs, 1), peak=HBM_PEAK_GBS, unit="GB/s", frac=round(gbs / HBM_PEAK_GBS, 4),
                         traffic=None, kernel="k_gemv_q6k", us_per_launch=round(us, 3), bytes_per_launch=nbytes)}))


def bench_hc(args, torch, capi, synth):
    """The layer together with the hyper-connection combine that consumes its output (four residual streams): the
    combine folded into the layer's last dispatch against the layer followed by the combine as a launch of its own.
    `--layers` different C2 layers per captured chain, router-selected experts."""
    H, F, k, E, NL, hc = 2048, 512, 10, args.experts, args.layers, 4
    layers, keep = build_stack(torch, synth, capi, NL, E, synth.BASE_SEED)
    scratch = C.c_void_p()
    capi.call("wd_moe_scratch_create", C.byref(scratch), H, F, E, k)
    rng = synth.rng_for(synth.BASE_SEED, 9300)
    d_x = torch.from_numpy(synth.rms_normed(rng, H)).cuda()
    d_out = torch.zeros(H, dtype=torch.float32, device="cuda")
    d_inject = torch.from_numpy(rng.normal(0, 1, hc).astype(np.float32)).cuda()
    res0 = torch.from_numpy(rng.normal(0, 1, (hc, H)).astype(np.float32)).cuda()
    d_res = res0.clone()
    stream = lambda: C.c_void_p(torch.cuda.current_stream().cuda_stream)
    vp = lambda t: C.c_void_p(t.data_ptr())

    def folded(i):
        capi.call("wd_moe_layer_hc_f32", C.byref(layers[i % NL]), vp(d_x), vp(d_out), vp(d_res), vp(d_inject), hc, 0, scratch, 0, stream())

    def apart(i):
        capi.call("wd_moe_layer_f32", C.byref(layers[i % NL]), vp(d_x), vp(d_out), scratch, 0, stream())
        capi.call("wd_hc_combine_f32", vp(d_res), vp(d_out), vp(d_inject), H, hc, 0, stream())

    results = {}
    for name, fn in (("folded", folded), ("apart", apart)):
        d_res.copy_(res0)
        for i in range(NL):
            fn(i)
        torch.cuda.synchronize()
        results[name + "_residual"] = d_res.clone()
        results[name] = graph_period_us(torch, fn, NL, 50)
    same = bool(torch.equal(results["folded_residual"].view(torch.int32), results["apart_residual"].view(torch.int32)))
    ok = same and bool(torch.isfinite(d_res).all().item()) and capi.load().wd_moe_scratch_status(scratch) == 0
    note("layer + combine: folded %.2f us, apart %.2f us per layer" % (results["folded"], results["apart"]))
    nbytes = 27697152 + 2 * hc * H * 4   # the C2 layer plus the residual streams read and written
    print(json.dumps({
        "metric": "MoE layer + hyper-connection combine, batch=1: microseconds per layer", "value": round(results["folded"], 3),
        "unit": "us", "n_gpus": 1, "higher_is_better": False, "vs_baseline": None,
        "dtype": "int8 dot products, f32 accumulate", "data": "synthetic",
        "config": {"workload": "C2 layer (512 experts, top-10, IQ3_S/Q8_0, shared expert) + combine into 4 residual streams",
                   "layers": NL, "combine_as_its_own_launch_us": round(results["apart"], 3), "same_bits": same, "ok": ok},
        "roofline": dict(bound="hbm", achieved=round(nbytes / results["folded"] / 1e3, 1), peak=HBM_PEAK_GBS, unit="GB/s",
                         frac=round(nbytes / results["folded"] / 1e3 / HBM_PEAK_GBS, 4), traffic=None,
                         kernel="k_layer_ab + k_layer_c", us_per_launch=round(results["folded"], 3), bytes_per_launch=nbytes)}))


def bench_c0(args, torch, capi, synth):
    """The single-layer parity workload at stack depth: the 64-expert top-8 layer with Q8_0 gate/up/down and no shared expert
    (hidden 2048, ffn 512), `--layers` independent layers chained as in the headline workload, router-selected.  Up to 64
    layers run as one resident launch (`--path per-layer`: two dispatches per layer)."""
    H, F, k, E, NL = 2048, 512, 8, 64, args.layers
    g = torch.Generator(device="cuda")
    g.manual_seed(synth.BASE_SEED + 5)
    rb_h, rb_f = synth.row_bytes(synth.Q8_0, H), synth.row_bytes(synth.Q8_0, F)

    def q8(rows, cols):
        nb = rows * (cols // 32)
        t = torch.randint(-127, 128, (nb * 34,), dtype=torch.int8, device="cuda", generator=g).view(torch.uint8)
        d = (torch.randn(nb, device="cuda", generator=g).abs() * (0.02 / 127.0)).half()
        t.view(-1, 34)[:, 0:2] = d.view(torch.uint8).view(-1, 2)
        return t

    layers, keep = (capi.MoeLayer * NL)(), []
    for l in range(NL):
        t = dict(router=torch.randn(E, H, device="cuda", generator=g) * 0.02, gate=q8(E * F, H), up=q8(E * F, H),
                 down=q8(E * H, F))
        keep.append(t)
        d = layers[l]
        d.hidden, d.expert_ffn, d.n_experts, d.top_k, d.expert_scale = H, F, E, k, 1.0
        d.gate_type = d.up_type = d.down_type = synth.Q8_0
        for name, tensor in t.items():
            setattr(d, name, tensor.data_ptr())
        d.gate_stride = d.up_stride = F * rb_h
        d.down_stride = H * rb_f
    scratch = C.c_void_p()
    capi.call("wd_moe_scratch_create", C.byref(scratch), H, F, E, k)
    rng = synth.rng_for(synth.BASE_SEED, 9200)
    d_x = torch.from_numpy(synth.rms_normed(rng, H)).cuda()
    d_out = torch.zeros(H, dtype=torch.float32, device="cuda")

    per_layer = args.path == "per-layer"

    def launch(_i):
        capi.call("wd_moe_stack_f32", layers, NL, C.c_void_p(d_x.data_ptr()), C.c_void_p(d_out.data_ptr()), scratch, None,
                  RESIDUAL_SCALE, 0x200 if per_layer else 0, C.c_void_p(torch.cuda.current_stream().cuda_stream))

    us = graph_period_us(torch, launch, 1, 50) / NL
    ok = bool(torch.isfinite(d_x).all().item()) and capi.load().wd_moe_scratch_status(scratch) == 0
    nbytes = E * H * 4 + k * (2 * F * rb_h + H * rb_f)
    assert nbytes == 27262976
    print(json.dumps({
        "metric": "MoE layer batch=1 decode, 64 experts top-8 all Q8_0: us per layer", "value": round(us, 2), "unit": "us",
        "n_gpus": 1, "higher_is_better": False, "vs_baseline": None,
        "dtype": "int8 dot products (Q8_0 weights x Q8_0 activations), f32 accumulate", "data": "synthetic",
        "config": {"workload": "C0: %d chained layers of hidden 2048, 64 experts, top-8, ffn 512, Q8_0 gate/up/down, "
                               "router-selected, batch=1, HIP-graph replay" % NL,
                   "layers": NL, "bytes_per_layer": nbytes, "tok_s_at_%d_layers" % NL: round(1e6 / (us * NL), 1), "valid": ok},
        "roofline": dict(bound="hbm", achieved=round(nbytes / us / 1e3, 1), peak=HBM_PEAK_GBS, unit="GB/s",
                         frac=round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4), traffic=None,
                         kernel="k_stack_resident<Q8_0> (one launch for the %d layers)" % NL if NL <= 64 and not per_layer else
                                "whole layer (k_layer_ab<Q8_0>, k_layer_c)")}))
    if not ok:
        sys.exit(1)


def bench_tokens(args, torch, capi, synth):
    """Speculative-verify batch: T correlated tokens through each of the C2 layers in one
    pass that reads every selected expert once, against T one-token passes over the same layers.  The router picks
    the experts; the tokens are mixed from a common direction so that their top-10 sets overlap by about half."""
    H, F, k, E, NL, T = 2048, 512, 10, args.experts, args.layers, args.tokens
    layers, keep = build_stack(torch, synth, capi, NL, E, synth.BASE_SEED)
    rng = synth.rng_for(synth.BASE_SEED, 9104)
    base = rng.normal(0, 1, H)
    xs = np.stack([TOKEN_MIX * base + (1.0 - TOKEN_MIX) * rng.normal(0, 1, H) for _ in range(T)])
    xs = (xs / np.sqrt((xs ** 2).mean(axis=1, keepdims=True))).astype(np.float32)
    d_x = torch.from_numpy(xs).cuda()
    d_out = torch.zeros((T, H), dtype=torch.float32, device="cuda")
    d_out1 = torch.zeros((T, H), dtype=torch.float32, device="cuda")
    scr = []
    for _ in range(T):
        h = C.c_void_p()
        capi.call("wd_moe_scratch_create", C.byref(h), H, F, E, k)
        scr.append(h)
    arr = (C.c_void_p * T)(*[h.value for h in scr])
    stream = lambda: C.c_void_p(torch.cuda.current_stream().cuda_stream)
    lib = capi.load()

    def batch(l):
        capi.call("wd_moe_layer_tokens_f32", C.byref(layers[l]), C.c_void_p(d_x.data_ptr()), C.c_void_p(d_out.data_ptr()), T, arr,
                  0, stream())

    def serial(l):
        for t in range(T):
            capi.call("wd_moe_layer_f32", C.byref(layers[l]), C.c_void_p(d_x[t].data_ptr()), C.c_void_p(d_out1[t].data_ptr()),
                      scr[t], 0, stream())

    unions, same = [], True
    for l in range(NL):                       # untimed: union sizes, and the two ways must agree bit for bit
        batch(l)
        torch.cuda.synchronize()
        ids = np.empty((T, k), np.int32)
        for t in range(T):
            capi.call("wd_memcpy_d2h", ids[t].ctypes.data_as(C.c_void_p), C.c_void_p(lib.wd_moe_scratch_ids(scr[t])), 4 * k, None)
        unions.append(len(set(ids.reshape(-1).tolist())))
        serial(l)
        torch.cuda.synchronize()
        same = same and bool(torch.equal(d_out.view(torch.int32), d_out1.view(torch.int32)))
    note("union of the %d top-%d sets: mean %.1f experts (min %d, max %d); batch == serial bit for bit: %s"
         % (T, k, np.mean(unions), min(unions), max(unions), same))
    if not same:
        print("bench.py: the token batch differs from the one-token passes", file=sys.stderr)
        sys.exit(1)
    reps = 10
    us_batch = graph_period_us(torch, batch, NL, reps)
    us_serial = graph_period_us(torch, serial, NL, reps)
    q8h, q8f, iq3h = synth.row_bytes(synth.Q8_0, H), synth.row_bytes(synth.Q8_0, F), synth.row_bytes(synth.IQ3_S, H)
    per_expert = 2 * F * iq3h + H * q8f
    fixed = E * H * 4 + H * 4 + 2 * F * q8h + H * q8f
    union_bytes = np.mean(unions) * per_expert + fixed
    serial_bytes = T * (k * per_expert + fixed)
    print(json.dumps({
        "metric": "speculative-verify pass of %d tokens through one MoE layer: us per layer" % T,
        "value": round(us_batch, 2), "unit": "us", "n_gpus": 1, "higher_is_better": False, "vs_baseline": None,
        "dtype": "int8 dot products (IQ3_S/Q8_0 weights x Q8_K/Q8_0 activations), f32 accumulate", "data": "synthetic",
        "config": {"workload": "C4: %d tokens (router-selected, correlated inputs) through each of %d C2 layers, "
                               "each selected expert read once per pass" % (T, NL),
                   "tokens": T, "layers": NL, "experts": E, "top_k": k, "union_mean": round(float(np.mean(unions)), 2),
                   "union_min": min(unions), "union_max": max(unions), "batch_equals_serial_bitwise": same,
                   "us_per_layer_batch": round(us_batch, 2), "us_per_layer_serial": round(us_serial, 2),
                   "speedup_vs_serial": round(us_serial / us_batch, 3),
                   "union_bytes_per_layer": int(union_bytes), "serial_bytes_per_layer": int(serial_bytes)},
        "roofline": dict(bound="hbm", achieved=round(union_bytes / us_batch / 1e3, 1), peak=HBM_PEAK_GBS, unit="GB/s",
                         frac=round(union_bytes / us_batch / 1e3 / HBM_PEAK_GBS, 4), traffic=None,
                         kernel="whole pass (k_tokens_a, k_tokens_b, k_tokens_c)")}))


def main():
    if len(sys.argv) >= 6 and sys.argv[1] == "--cpu-child":
        cpu_child(float(sys.argv[2]), int(sys.argv[3]), sys.argv[4], sys.argv[5])
        return
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the MoE decode hot path of the "
              "reference is single-GPU); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    from warpdecode_amd import capi, synth

    torch.cuda.set_device(0)
    capi.call("wd_init", 0)
    H, F, k, E, NL = 2048, 512, 10, args.experts, args.layers
    if args.mode == "q4-sweep":
        return bench_q4_sweep(args, torch, capi, synth)
    if args.mode == "q8-sweep":
        return bench_q8_sweep(args, torch, capi, synth)
    if args.mode == "q8-batch":
        return bench_q8_batch(args, torch, capi, synth)
    if args.mode == "c0":
        return bench_c0(args, torch, capi, synth)
    if args.mode == "model-layer":
        return bench_model_layer(args, torch, capi, synth)
    if args.mode == "q6k-head":
        return bench_q6k_head(args, torch, capi, synth)
    note("generating %d layers x %d experts on the device" % (NL, E))
    if args.mode == "tokens":
        return bench_tokens(args, torch, capi, synth)
    if args.mode == "lru":
        print(json.dumps(bench_lru(args, torch, capi, synth)))
        return
    if args.mode == "hc":
        return bench_hc(args, torch, capi, synth)
    layers, keep = build_stack(torch, synth, capi, NL, E, synth.BASE_SEED)
    torch.cuda.synchronize()
    note("weights ready (%.1f GB allocated)" % (torch.cuda.memory_allocated() / 1e9))
    scratch = C.c_void_p()
    capi.call("wd_moe_scratch_create", C.byref(scratch), H, F, E, k)

    total_steps = args.warmup + args.steps
    rng = synth.rng_for(synth.BASE_SEED, 9001)
    perms = [rng.permutation(E) for _ in range(NL)]
    trace = np.stack([np.stack([synth.zipf_ids(rng, E, k, 1.1, perms[l]) for l in range(NL)])
                      for _ in range(total_steps)]).astype(np.int32)           # [steps][layers][k]
    xs = np.stack([synth.rms_normed(rng, H) for _ in range(total_steps)])
    # A token's input is one piece of device memory, the activation followed by its routing trace, so that a step brings
    # its input in with one copy.
    inputs = np.concatenate([xs.view(np.int32), trace.reshape(total_steps, NL * k)], axis=1)
    d_inputs = torch.from_numpy(inputs).cuda()
    d_input = torch.zeros(H + NL * k, dtype=torch.int32, device="cuda")
    d_x, d_trace = d_input[:H].view(torch.float32), d_input[H:].view(NL, k)
    d_out = torch.zeros(H, dtype=torch.float32, device="cuda")
    trace_ptr = C.c_void_p(d_trace.data_ptr()) if args.routing == "zipf" else None

    def bring_in(i):
        d_input.copy_(d_inputs[i % total_steps], non_blocking=True)

    PER_LAYER = 0x200   # WD_MOE_PER_LAYER
    stack_flags = STACK_FLAGS | (PER_LAYER if args.path == "per-layer" else 0)

    def launch_stack(flags=None):
        capi.call("wd_moe_stack_f32", layers, NL, C.c_void_p(d_x.data_ptr()), C.c_void_p(d_out.data_ptr()), scratch,
                  trace_ptr, RESIDUAL_SCALE, stack_flags if flags is None else flags,
                  C.c_void_p(torch.cuda.current_stream().cuda_stream))

    def captured(fn, one_launch=False):
        """fn() warmed on a side stream, then captured into a HIP graph (None when it is to be launched eagerly)."""
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        if args.no_graph or args.graph == "off" or (args.graph == "auto" and one_launch):
            return None
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            fn()
        return g

    def first_token(flags, n_layers=NL):
        """x and out (host copies) of token 0 through the first n_layers layers by the given form of the stack."""
        bring_in(0)
        capi.call("wd_moe_stack_f32", layers, n_layers, C.c_void_p(d_x.data_ptr()), C.c_void_p(d_out.data_ptr()), scratch,
                  trace_ptr, RESIDUAL_SCALE, flags, C.c_void_p(torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        return d_x.cpu().numpy().copy(), d_out.cpu().numpy().copy()

    # The launch that is timed, against the other form of the stack on the same token: all layers at full width, bit for bit.
    got, alt = first_token(stack_flags), first_token(stack_flags ^ PER_LAYER)
    forms_agree = all(np.array_equal(a.view(np.uint32), b.view(np.uint32)) for a, b in zip(got, alt))
    note("token 0 through %d layers: resident launch and per-layer dispatches bit-identical: %s" % (NL, forms_agree))
    if not forms_agree:
        print("bench.py: the two forms of the stack disagree on token 0", file=sys.stderr)
        sys.exit(1)
    oracle_checked = None
    if args.check:
        # the measured form of the stack on layer 0 alone against the CPU oracle (ids from the trace, the router's weights)
        from oracle import pyoracle
        L0 = layer_dict(torch, synth, keep[0], E)
        if trace_ptr is None:
            want, _ = pyoracle.moe_layer(L0, xs[0])
        else:
            _, wts = pyoracle.route(pyoracle.router_logits(L0["router"], xs[0]), k)
            want, _ = pyoracle.moe_layer(L0, xs[0], ids=trace[0][0], weights=wts)
        want_x = (xs[0] + (want * np.float32(RESIDUAL_SCALE)).astype(np.float32)).astype(np.float32)
        got_x, got_out = first_token(stack_flags, 1)
        oracle_checked = bool(np.array_equal(got_out.view(np.uint32), want.view(np.uint32)) and
                              np.array_equal(got_x.view(np.uint32), want_x.view(np.uint32)))
        print("check: layer 0 through the measured form of the stack bit-identical to the CPU oracle: %s" % oracle_checked,
              file=sys.stderr)
        if not oracle_checked:
            sys.exit(1)

    note("inputs and routing trace ready")
    graph = captured(launch_stack, one_launch=args.path == "resident")

    note("launch mode: %s" % ("eager" if graph is None else "hip-graph replay"))

    def step(i):
        bring_in(i)
        if graph is not None:
            graph.replay()
        else:
            launch_stack()

    def timed_region(first):
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
        for i in range(args.steps):
            step(first + i)
        ev1.record()
        torch.cuda.synchronize()
        return ev0.elapsed_time(ev1) / args.steps

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    note("warm-up done, timing %d steps" % args.steps)
    t0 = time.perf_counter()
    ms_per_step = timed_region(args.warmup)
    wall = time.perf_counter() - t0
    tok_s = 1000.0 / ms_per_step
    finite = bool(torch.isfinite(d_x).all().item())
    waits_ok = capi.load().wd_moe_scratch_status(scratch) == 0   # no bounded wait inside a dispatch ran out
    note("timed region done: %.3f ms/step" % ms_per_step)
    if not (finite and waits_ok):
        print("bench.py: invalid run (finite=%s, in-dispatch waits ok=%s)" % (finite, waits_ok), file=sys.stderr)
        sys.exit(1)
    repeats = sorted([ms_per_step] + [timed_region(args.warmup + (j + 1) * 7) for j in range(args.repeats)])
    spread = dict(min=round(repeats[0], 4), median=round(repeats[len(repeats) // 2], 4), max=round(repeats[-1], 4),
                  regions=len(repeats))
    note("spread of %d timed regions: %s" % (len(repeats), spread))

    # Algorithmic bytes of the two dispatches of one layer (weights only, as the workload prices them):
    #   AB router f32 [E][H] + the shared expert's gate vector + its Q8_0 gate and up matrices
    #      + gate and up (IQ3_S) of the k selected experts
    #   C  down (Q8_0) of the k selected experts and of the shared expert
    q8h, q8f, iq3h = synth.row_bytes(synth.Q8_0, H), synth.row_bytes(synth.Q8_0, F), synth.row_bytes(synth.IQ3_S, H)
    alg = {"k_layer_ab": E * H * 4 + H * 4 + 2 * F * q8h + k * 2 * F * iq3h, "k_layer_c": (k + 1) * H * q8f}
    bytes_per_layer = sum(alg.values())
    assert E != 512 or bytes_per_layer == 27697152
    bytes_per_step = bytes_per_layer * NL

    def period_ms(runner, reps):
        for _ in range(3):
            runner()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            runner()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps

    per_kernel, reps, router_driven = {}, 20, None
    step(0)
    if args.path == "resident":
        # the figures below are named for k_stack_resident: make sure that it is what the library launches on this device
        # (it takes the dispatches per layer, silently, where the 512 workgroups cannot all be resident at once)
        lib = capi.load()
        sites = [i for i in range(64) if b"resident" in lib.wd_profile_site_name(i)]
        capi.call("wd_profile_enable", 1)
        capi.call("wd_profile_reset")
        bring_in(0)
        launch_stack()
        torch.cuda.synchronize()
        capi.call("wd_profile_flush_token")
        st, seen = capi.ProfileSiteStat(), C.c_ulonglong()
        capi.call("wd_profile_site", sites[0], C.byref(st), C.byref(seen))
        capi.call("wd_profile_enable", 0)
        capi.call("wd_profile_reset")
        if len(sites) != 1 or st.calls != 1:
            raise SystemExit("bench.py: the stack did not run as one resident launch on this device (--path per-layer measures the dispatches per layer)")
        # The dominant kernel is the step itself: one launch of k_stack_resident covers the 48 layers.  Timed live with HIP
        # events on the launch stream over `reps` launches (graph replays) without the input copies of step().
        # (fresh input and routing trace before every launch, as in the timed region; the events bracket the launch alone)
        run_it = graph.replay if graph is not None else launch_stack
        pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
        for j, (e0, e1) in enumerate(pairs):
            bring_in(j)
            e0.record()
            run_it()
            e1.record()
        torch.cuda.synchronize()
        us = sum(e0.elapsed_time(e1) for e0, e1 in pairs) / reps * 1e3
        per_kernel["k_stack_resident"] = dict(us_per_launch=round(us, 2), bytes_per_launch=bytes_per_step,
                                              achieved=round(bytes_per_step / (us * 1e-6) / 1e9, 1), layers_per_launch=NL,
                                              us_per_layer=round(us / NL, 3))
        # the same step as two dispatches per layer, for comparison
        g2 = captured(lambda: launch_stack(STACK_FLAGS | PER_LAYER))
        run_alt = g2.replay if g2 is not None else (lambda: launch_stack(STACK_FLAGS | PER_LAYER))

        def alt_step(j):
            bring_in(j)
            run_alt()
        for j in range(4):
            alt_step(j)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for j in range(reps):
            alt_step(4 + j)
        e1.record()
        torch.cuda.synchronize()
        per_kernel["per_layer_dispatches"] = dict(ms_per_step=round(e0.elapsed_time(e1) / reps, 4))
        dominant = "k_stack_resident"
        if trace_ptr is not None:
            # the same launch with nothing known ahead: every layer's ids come from its own router, inside the launch
            def router_stack():
                capi.call("wd_moe_stack_f32", layers, NL, C.c_void_p(d_x.data_ptr()), C.c_void_p(d_out.data_ptr()), scratch,
                          None, RESIDUAL_SCALE, STACK_FLAGS, C.c_void_p(torch.cuda.current_stream().cuda_stream))
            g3 = captured(router_stack, one_launch=True)
            run_router = g3.replay if g3 is not None else router_stack
            for j in range(4):
                bring_in(j)
                run_router()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for j in range(args.steps):
                bring_in(4 + j)
                run_router()
            e1.record()
            torch.cuda.synchronize()
            ms_router = e0.elapsed_time(e1) / args.steps
            router_driven = dict(ms_per_step=round(ms_router, 4), tok_s=round(1000.0 / ms_router, 2), steps=args.steps,
                                 finite=bool(torch.isfinite(d_x).all().item()),
                                 in_dispatch_waits_ok=capi.load().wd_moe_scratch_status(scratch) == 0)
            note("router-selected experts, same launch: %s" % router_driven)
    else:
        # Per-kernel launch time, live: the stack is replayed with one dispatch per layer only (the other left out), so
        # the timed region is a chain of NL launches of that one kernel over NL layers' weights.  The period includes
        # the gap between two dependent launches on a stream, which a profiler's begin-to-end time omits.
        only = {"k_layer_ab": 0x30, "k_layer_c": 0x40}
        for name, flag in only.items():
            def chain():
                launch_stack(flag | CHAIN_FLAGS | PER_LAYER)
            g1 = captured(chain)
            us = period_ms(g1.replay if g1 is not None else chain, reps) * 1e3 / NL
            per_kernel[name] = dict(us_per_launch=round(us, 3), bytes_per_launch=alg[name],
                                    achieved=round(alg[name] / (us * 1e-6) / 1e9, 1))
        dominant = max(per_kernel, key=lambda n: per_kernel[n]["us_per_launch"])
    note("per-kernel launch periods: %s; dominant: %s" % (per_kernel, dominant))
    traffic = recorded_traffic(dominant)
    dom = per_kernel[dominant]
    whole = bytes_per_step / (ms_per_step * 1e-3) / 1e9
    roofline = dict(bound="hbm", achieved=dom["achieved"], peak=HBM_PEAK_GBS, unit="GB/s",
                    frac=round(dom["achieved"] / HBM_PEAK_GBS, 4), traffic=traffic,
                    kernel=dominant, us_per_launch=dom["us_per_launch"], bytes_per_launch=dom["bytes_per_launch"],
                    kernels=per_kernel,
                    whole_step=dict(achieved=round(whole, 1), frac=round(whole / HBM_PEAK_GBS, 4),
                                    bytes_per_step=bytes_per_step))

    # A plain copy of known size, so that a counter run of this command can scale FETCH_SIZE / WRITE_SIZE.
    cal_src = torch.empty(64 << 20, dtype=torch.float32, device="cuda").normal_()
    cal_dst = torch.empty_like(cal_src)
    cal_dst.copy_(cal_src)
    torch.cuda.synchronize()
    del cal_src, cal_dst

    site_profile = None
    if args.site_profile > 0:
        # eager launches: a bracket on a capturing stream is not recorded.  One pass per form of the stack.
        import re
        site_profile = {}
        lib = capi.load()
        for form, flags in (("resident_launch", STACK_FLAGS), ("per_layer_dispatches", STACK_FLAGS | PER_LAYER)):
            capi.call("wd_profile_enable", 1)
            capi.call("wd_profile_reset")
            for j in range(args.site_profile):
                bring_in(j)
                launch_stack(flags)
                torch.cuda.synchronize()
                capi.call("wd_profile_flush_token")
            need = lib.wd_profile_report(None, 0)
            buf = C.create_string_buffer(need + 1)
            lib.wd_profile_report(buf, need + 1)
            capi.call("wd_profile_enable", 0)
            print("site profile, %s:\n%s" % (form, buf.value.decode()), file=sys.stderr, flush=True)
            site_profile[form] = {line.split()[1]: {key: float(v) for key, v in re.findall(r"([a-z/]+)=\s*([-0-9.]+)", line)}
                                  for line in buf.value.decode().splitlines()[1:]}

    out = {
        "metric": "MoE layer batch=1 decode: synthetic 48-layer tok/s (achieved HBM GB/s in roofline)",
        "value": round(tok_s, 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 dot products (IQ3_S/Q8_0 weights x Q8_K/Q8_0 activations), f32 accumulate",
        "data": "synthetic",
        "config": {"workload": "C3 mode A: %d-layer stack of the 512-expert top-10 IQ3_S/Q8_0 MoE layer "
                               "(hidden 2048, ffn 512, Q8_0 shared expert), batch=1, all experts resident in HBM"
                               % NL,
                   "layers": NL, "experts": E, "top_k": k, "routing": args.routing,
                   "launch": "eager" if graph is None else "hip-graph replay",
                   "path": "one resident launch per step" if args.path == "resident" else "two dispatches per layer",
                   "spread_ms_per_step": spread,
                   "bytes_per_token": bytes_per_step, "wall_s": round(wall, 3), "finite": finite,
                   "in_dispatch_waits_ok": waits_ok, "forms_bit_identical_on_token_0": forms_agree,
                   "layer_0_equals_cpu_oracle": oracle_checked, "router_selected_ids_same_launch": router_driven},
        "roofline": roofline,
    }
    if site_profile is not None:
        out["config"]["site_profile_ms_per_token"] = site_profile
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(args.cpu_seconds)
    if not args.no_mode_b and args.path == "resident" and E == 512 and NL == 48:
        # The same stack with its routed experts in pinned host memory behind the slot pool (a bounded run: the tokens
        # that warm the pool, then --steps tokens).  The resident stack's device copies are given up for it, so it runs last.
        del graph, g2
        try:
            b = bench_lru(args, torch, capi, synth, stack=(layers, keep))
            c = b["config"]
            out["mode_b"] = dict(tok_s=b["value"], ms_per_step=b["ms_per_step"], steps=b["steps"], hit_rate=c["hit_rate"],
                                 misses_per_token=c["misses_per_token"], host_link_bytes_per_token=c["host_link_bytes_per_token"],
                                 host_link_GBps=c["host_link_GBps"], host_ms_per_step=c["host_ms_per_step"], slots=c["slots"],
                                 slot_bytes=c["slot_bytes"], cache_gib=args.cache_gib, cache_warm_tokens=c["cache_warm_tokens"],
                                 source=c["source"], driver=c["driver"], launch=c["launch"], path=c["path"], finite=c["finite"],
                                 workload=c["workload"])
        except Exception as exc:      # e.g. the box refuses 49.5 GB of pinned host memory
            out["mode_b"] = dict(skipped="%s: %s" % (type(exc).__name__, exc))
        note("mode B: %s" % out["mode_b"])
    print(json.dumps(out))


if __name__ == "__main__":
    main()
