#!/usr/bin/env python3
"""Headline benchmark: examples/sec of forward + backward + EM on the 3072-variable HCLT
(K = 32, 256 categories, batch 4096) on one MI355X, with the dominant kernel's roofline
fraction and the CPU oracle timed beside it.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3_hclt3072_k32]

A step is one mini-batch EM iteration (pcm_em_step: stage batch, forward, backward,
statistics, parameter update) on a batch already resident in HBM.  Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "lvd-pg_amd"))

HBM_PEAK_GBS = 8000.0   # MI355X HBM3E, published
# the layered engine's byte count is what its kernels ask the caches for, not what must cross the HBM interface
REQUESTED_NOTE = ("bytes the circuit asks for edge by edge: 8 per (node, example) + 24 per (edge, example), a measure of the "
                  "work; sums that run as dense groups read a child's row once per group, and at this size most requests "
                  "are served by L2 and the last-level cache, so frac is not a fraction of HBM traffic")
# kernels the benchmark circuit runs (three children per node at most, K = 32: the lean set)
PHASE_MASK = {"forward": 2, "backward": 4, "statistics": 8}   # pcm_set_timing: time that phase's kernel only
KERNEL_NAMES = {"forward": "hclt_forward_lean_kernel<%d>", "backward": "hclt_backward_lean_kernel<%d, false>",
                "statistics": "hclt_stats_lean_kernel<%d>"}


def algorithmic_bytes(n_int, V, K, C, B):
    """Bytes the algorithm has to move per launch, per kernel.  A node-value or flow vector
    is K*4 bytes per (tree node, example); the whole step is priced at six of them per tree
    node (value written and read as a child going up, read twice going down, flow written
    once and read once).  They are booked where this implementation's kernels touch them, two
    per kernel: forward (value written, value read as a child), backward
    (children's values read, ratio vector written: a node's own value is not read going
    down), statistics (ratio vector read, children's values read to rebuild the edge
    weights).  The forward walk's second vector, the value read as a child, never leaves LDS in this
    implementation, so that kernel's own roofline entry counts the ONE vector that reaches HBM (the step's
    total keeps all six).  Each kernel also reads the batch (V*B bytes), the sum parameters (4 bytes per
    edge) and the leaf tables (4*V*K*C); statistics additionally writes both accumulators."""
    vec = K * 4 * B
    n_sum_edges = (n_int - 1) * K * K + K
    theta = 4 * n_sum_edges
    leaf = 4 * V * K * C
    fwd = n_int * 1 * vec + V * B + theta + leaf
    bwd = n_int * 2 * vec + V * B + theta + leaf
    stats = n_int * 2 * vec + V * B + 2 * theta + 2 * leaf
    return dict(forward=fwd, backward=bwd, statistics=stats,
                step=n_int * 6 * vec + V * B + 3 * theta + 5 * leaf)


def measured_traffic(workload, kernel):
    """HBM bytes per launch of `kernel` from the committed hardware-counter summary
    (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a copy of known size), or None."""
    path = os.path.join(ROOT, "profiles", f"hclt_em_step_{workload}_hbm_traffic.txt")
    try:
        for line in open(path):
            f = line.split()
            if len(f) == 4 and f[0] == "traffic_bytes" and f[1] == workload and f[2] == kernel:
                return float(f[3])
    except OSError:
        pass
    return None


def cpu_baseline(cfg, sample):
    """The oracle (a C port of the reference arithmetic, OpenMP over examples) on the
    first `sample` examples of the same batch: one full EM step."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import numpy as np
    import pc_oracle as O
    parent, K, C = cfg["parent"], cfg["K"], cfg["C"]
    ch, _ = O.clt_children(parent)
    theta = {v: cfg["theta"][v] for v in range(len(parent)) if ch[v]}
    fc = O.hclt_flat(parent, K, C, theta, cfg["leaf"])
    data = np.ascontiguousarray(cfg["data"][:sample])
    idx = np.arange(sample, dtype=np.int32)
    t0 = time.perf_counter()
    ll, *_ = O.em_step(fc, data, idx, 0.1, 0.9)
    dt = time.perf_counter() - t0
    return dict(value=sample / dt, unit="examples/s", cores=int(O.lib().orc_max_threads()), kind="port",
                sample=f"one EM step on the first {sample} examples of the batch, {dt:.1f} s"), ll


def _timed(torch, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def _patch_heads(P, parent, K, C, H, rng):
    """A patch circuit as the progressive-growing experiments build it: one HCLT body and H head
    sum nodes over the K products under its root (exps/progressive_growing/parallel_PG.jl:214-225),
    parameters drawn as `init_parameters(perturbation = 0.4)` draws them."""
    from pcmi355 import nodes as N
    body = P.hclt_pc(parent, C, K)
    heads = [N.summate(list(body.inputs)) for _ in range(H)]
    N.init_parameters(heads, perturbation=0.4, rng=rng)
    return heads


def secondary(args):
    """The other configurations (not the headline; same JSON shape).  c2: wide block kernels,
    priced against the fp32 matrix peak.  c4: layered engine, whose byte count is its own minimum:
    per example 4 bytes written per node and 8 read per edge going up; going down 4 written per
    node and 16 read per incoming edge.  c5: block-form queries."""
    import numpy as np
    import torch
    import pcmi355 as P
    from pcmi355 import workloads
    from pcmi355._lib import lib, check
    rng = np.random.default_rng(0)
    note = None
    out = {"n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "dtype": "f32", "data": "synthetic", "cpu_baseline": None}
    if args.workload == "c2_hclt48_k128":
        c2 = workloads.c2_config()
        V, K, C, B, data, parent, theta, leaf = (c2[k] for k in ("V", "K", "C", "B", "data", "parent", "theta", "leaf"))
        bpc = P.hclt_from_clt(parent, C, K)
        bpc.set_params(theta, leaf)
        d = torch.from_numpy(data).cuda()
        ll = torch.empty(B, device="cuda")
        dt = _timed(torch, lambda: check(lib.pcm_em_step(bpc.handle, d.data_ptr(), d.stride(0), d.stride(1), None, B,
                                                          0.0, 0.1, 0.9, ll.data_ptr())), args.steps, args.warmup)
        n_int = bpc.size("inner_tree_nodes")
        flops = 6.0 * K * K * B * n_int                      # three K x K contractions per (tree node, example)
        out.update(metric="examples/sec fwd+bwd+EM, 48-var HCLT K=128 (wide block kernels)", value=B / dt, unit="examples/s",
                   config={"workload": args.workload, "num_vars": V, "hidden": K, "categories": C, "batch": B,
                           "tree_inner_nodes": n_int})
        out["ms_per_step"] = dt * 1e3
        ach = flops / dt / 1e12
        out["roofline"] = {"bound": "mfma", "kernel": "whole step", "achieved": ach, "peak": 157.3, "unit": "TFLOP/s",
                           "frac": ach / 157.3, "traffic": None}
        print(json.dumps(out))
        return
    elif args.workload in ("c4_patch_multihead", "c4_patch_multihead_block"):
        V, K, C, H, B = 192, 32, 256, 128, 1024
        data = workloads.grf_images(B, 8, 8, 3, 3.0, 0.8, seed=1004)
        parent = workloads.chow_liu_parent(data)
        if args.workload.endswith("_block"):      # the same circuit on the block engine
            bpc, engine = P.multihead_hclt_from_clt(parent, C, K, H), "block engine"
            bpc.set_params(*workloads.init_params(parent, K, C, 1104, kind="dirichlet"))     # heads stay uniform
        else:
            bpc, engine = P.CuMultiHeadBitsProbCircuit(_patch_heads(P, parent, K, C, H, rng), V), "layered engine"
        mask = np.zeros((B, H), np.float32)
        mask[np.arange(B), rng.integers(0, H, size=B)] = 1.0
        d = torch.from_numpy(data).cuda()
        hm = torch.from_numpy(mask).cuda().t().contiguous()
        ll = torch.empty(B, device="cuda")

        def step():
            check(lib.pcm_flows(bpc.handle, d.data_ptr(), d.stride(0), d.stride(1), None, B, 0.0, hm.data_ptr(), ll.data_ptr()))
            check(lib.pcm_em_update(bpc.handle, 0.1, 0.9))
        dt = _timed(torch, step, args.steps, args.warmup)
        nn, ne = bpc.num_nodes(), bpc.num_edges()
        algo = B * (8 * nn + 24 * ne)
        note = REQUESTED_NOTE
        if engine == "block engine":   # block form: six K-vectors per tree node and example, the mask read going up and down
            algo = algorithmic_bytes(bpc.size("inner_tree_nodes"), V, K, C, B)["step"] + 2 * 4 * H * B
            note = None
        out.update(metric="examples/sec fwd+bwd+EM, 192-var patch circuit K=32 with 128 heads (%s)" % engine,
                   value=B / dt, unit="examples/s",
                   config={"workload": args.workload, "num_vars": V, "hidden": K, "categories": C, "heads": H,
                           "batch": B, "nodes": nn, "edges": ne})
    elif args.workload == "c5_variational":
        cfg = workloads.make_config("c3_hclt3072_k32")
        V, K, C, B = cfg["V"], cfg["K"], cfg["C"], cfg["B"]
        p = P.hclt_from_clt(cfg["parent"], C, K)
        p.set_params(cfg["theta"], cfg["leaf"])
        q = P.hclt_from_clt(cfg["parent"], C, K)
        q.set_params(*workloads.init_params(cfg["parent"], K, C, 4243, kind="dirichlet"))
        n_inner = p.size("inner_tree_nodes")
        gen = torch.Generator(device="cuda").manual_seed(5)
        node_noise = -torch.log(-torch.log(torch.rand((B, n_inner * K), device="cuda", generator=gen).clamp_(1e-10, 1 - 1e-7)))
        leaf_noise = torch.empty((B, V, C), device="cuda")
        for s0 in range(0, B, 512):
            leaf_noise[s0:s0 + 512] = -torch.log(-torch.log(torch.rand((512, V, C), device="cuda", generator=gen).clamp_(1e-10, 1 - 1e-7)))
        P.kld(p, q)                                                   # builds the tables
        t_kld = _timed(torch, lambda: P.kld(p, q), args.steps, 1)
        t_grad = _timed(torch, lambda: P.kld_backward(p, q, device=True), args.steps, 1)
        t_samp = _timed(torch, lambda: P.sample(p, node_noise, leaf_noise), max(1, args.steps // 4), 1)
        n_sum = p.num_inner_params()
        g1, _ = P.kld_backward(p, q, device=True)
        dp = torch.from_numpy(P.vectorize_parameters(p)[:n_sum].copy()).cuda()
        dm, dv = torch.zeros_like(dp), torch.zeros_like(dp)
        tt = [0]

        def adam():
            tt[0] += 1
            P.adam_step(p, g1, dp, dm, dv, lr=1e-4, t=tt[0])
        t_adam = _timed(torch, adam, args.steps, 1)
        soft_out = torch.empty((B, V, C), device="cuda")
        t_soft = _timed(torch, lambda: check(lib.pcm_sample_soft(p.handle, node_noise.data_ptr(), 0.5, B, soft_out.data_ptr())),
                        max(1, args.steps // 4), 1)
        del soft_out, node_noise, leaf_noise
        # the same queries on a matrix of 64 parameter rows (one parameter vector per example, as the
        # variational models call them): rows of p's parameters against rows of q's
        R = 64
        n_par = p.num_parameters()
        pv = torch.from_numpy(P.vectorize_parameters(p)).cuda()
        qv = torch.from_numpy(P.vectorize_parameters(q)).cuda()
        m1 = pv.repeat(R, 1)
        m2 = qv.repeat(R, 1)
        m1 += 0.01 * torch.randn((R, 1), device="cuda", generator=gen)      # rows differ (values only matter for the clock)
        klr = P.kld(p, m1, m2)
        t_kld_rows = _timed(torch, lambda: P.kld(p, m1, m2), max(1, args.steps // 4), 1)
        t_grad_rows = _timed(torch, lambda: P.kld_backward(p, m1, m2), max(1, args.steps // 4), 1)
        soft_rows = None
        t_soft_rows = _timed(torch, lambda: P.gumbel_sample_rows(p, m1, temperature=1.0), max(1, args.steps // 4), 1)
        og = torch.randn((R, V, C), device="cuda", generator=gen)
        t_soft_back_rows = _timed(torch, lambda: P.gumbel_sample_backward_rows(p, m1, og, temperature=1.0), max(1, args.steps // 4), 1)
        del og
        rows_bytes = {"kld_rows": 2 * 4 * R * n_par, "kld_backward_rows": 5 * 4 * R * n_par}
        del m1, m2, klr
        dt = t_samp
        algo = 4 * B * (n_inner * K + V * C)                           # the noise tensors, read once
        out.update(metric="samples/sec Gumbel-max from supplied noise, 3072-var HCLT K=32",
                   value=B / t_samp, unit="samples/s",
                   config={"workload": args.workload, "num_vars": V, "hidden": K, "categories": C, "batch": B},
                   queries_ms={"kld": t_kld * 1e3, "kld_backward_dev": t_grad * 1e3, "adam_step": t_adam * 1e3,
                               "sample": t_samp * 1e3, "gumbel_sample_relaxed_T0.5": t_soft * 1e3,
                               "kld_rows_R64": t_kld_rows * 1e3, "kld_backward_rows_R64": t_grad_rows * 1e3,
                               "gumbel_sample_rows_R64_no_gumbel": t_soft_rows * 1e3,
                               "gumbel_sample_backward_rows_R64_no_gumbel": t_soft_back_rows * 1e3},
                   rows_gbs={"kld_rows_R64": rows_bytes["kld_rows"] / t_kld_rows / 1e9,
                             "kld_backward_rows_R64": rows_bytes["kld_backward_rows"] / t_grad_rows / 1e9})
    elif args.workload == "c4_patch_x8_streams":
        # eight independent patch circuits (C4 has 64), each queued on one of four streams: the layered engine's
        # per-layer launches are small, so circuits overlap on the device
        V, K, C, H, B, NC, NS = 192, 32, 256, 128, 1024, 8, 4
        data = workloads.grf_images(B, 8, 8, 3, 3.0, 0.8, seed=1004)
        parent = workloads.chow_liu_parent(data)
        heads = _patch_heads(P, parent, K, C, H, rng)
        circs = [P.CuMultiHeadBitsProbCircuit(heads, V) for _ in range(NC)]
        mask = np.zeros((B, H), np.float32)
        mask[np.arange(B), rng.integers(0, H, size=B)] = 1.0
        d = torch.from_numpy(data).cuda()
        hm = torch.from_numpy(mask).cuda().t().contiguous()
        lls = [torch.empty(B, device="cuda") for _ in range(NC)]
        streams = [torch.cuda.Stream() for _ in range(NS)]
        torch.cuda.synchronize()
        for i, c in enumerate(circs):
            check(lib.pcm_set_stream(c.handle, streams[i % NS].cuda_stream))

        def step():
            for c, ll in zip(circs, lls):
                check(lib.pcm_flows(c.handle, d.data_ptr(), d.stride(0), d.stride(1), None, B, 0.0, hm.data_ptr(), ll.data_ptr()))
                check(lib.pcm_em_update(c.handle, 0.1, 0.9))
        dt = _timed(torch, step, args.steps, args.warmup)
        nn, ne = circs[0].num_nodes(), circs[0].num_edges()
        algo = NC * B * (8 * nn + 24 * ne)
        note = REQUESTED_NOTE
        out.update(metric="examples/sec fwd+bwd+EM over 8 independent 192-var K=32 128-head patch circuits on 4 streams",
                   value=NC * B / dt, unit="examples/s",
                   config={"workload": args.workload, "circuits": NC, "streams": NS, "num_vars": V, "hidden": K,
                           "categories": C, "heads": H, "batch": B})
    elif args.workload == "c4_patch_x16_as_one":
        # sixteen patch circuits over sixteen blocks of 192 variables compiled as ONE multi-head circuit (2048 heads):
        # every layer launch then carries the nodes of all sixteen, which is the layered engine with the device full
        from pcmi355 import nodes as N
        V, K, C, H, B, NC = 192, 32, 256, 128, 1024, 16
        data = workloads.grf_images(B, 8, 8, 3, 3.0, 0.8, seed=1004)
        parent = workloads.chow_liu_parent(data)
        heads = []
        for c in range(NC):
            hs = _patch_heads(P, parent, K, C, H, rng)
            for n in N.linearize(hs):
                if n.kind == N.INPUT:
                    n.var += c * V
            heads += hs
        bpc = P.CuMultiHeadBitsProbCircuit(heads, NC * V)
        mask = np.zeros((NC * H, B), np.float32)
        for c in range(NC):
            mask[c * H + rng.integers(0, H, size=B), np.arange(B)] = 1.0
        d = torch.from_numpy(np.tile(data, (1, NC))).cuda()
        hm = torch.from_numpy(mask).cuda()
        ll = torch.empty(B, device="cuda")

        def step():
            check(lib.pcm_flows(bpc.handle, d.data_ptr(), d.stride(0), d.stride(1), None, B, 0.0, hm.data_ptr(), ll.data_ptr()))
            check(lib.pcm_em_update(bpc.handle, 0.1, 0.9))
        dt = _timed(torch, step, args.steps, args.warmup)
        nn, ne = bpc.num_nodes(), bpc.num_edges()
        algo = B * (8 * nn + 24 * ne)
        note = REQUESTED_NOTE
        out.update(metric="examples/sec fwd+bwd+EM over 16 192-var K=32 128-head patch circuits compiled as one circuit "
                          "(layered engine); an example counts once per circuit",
                   value=NC * B / dt, unit="examples/s",
                   config={"workload": args.workload, "circuits": NC, "num_vars": V, "hidden": K, "categories": C,
                           "heads": H, "batch": B, "nodes": nn, "edges": ne})
    elif args.workload in ("c4_full", "c4_full_handles"):
        # C4 as a whole: 64 x 64 x 3 images cut into 64 patches of 8 x 8 x 3; one 192-variable K = 32 circuit with 128
        # cluster heads per patch and the K = 64 top-level HCLT over the 64 cluster ids.  c4_full: the 64 patch
        # circuits as ONE forest handle over the 12288 pixels (one launch per kernel for all of them);
        # c4_full_handles: a handle per patch circuit, queued on 32 streams.
        c4 = workloads.c4_config()
        V, K, C, H, B, NP, NS = c4["V"], c4["K"], c4["C"], c4["H"], c4["B"], c4["patches"], 32
        flat, cluster, pvars, parents, params = c4["data"], c4["cluster"], c4["pvars"], c4["parents"], c4["params"]
        top = P.hclt_from_clt(c4["top_parent"], H, 64)
        top.set_params(*c4["top_params"])
        dtop = torch.from_numpy(cluster).cuda()
        ll_top = torch.empty(B, device="cuda")
        n_int = [int((np.bincount(par[par >= 0], minlength=V) > 0).sum()) for par in parents]
        if args.workload == "c4_full":
            forest = P.hclt_forest_from_clts(c4["fparent"], C, K, H)         # heads stay uniform
            forest.set_params(c4["theta"], c4["leaf"])
            dmask = torch.from_numpy(c4["mask"]).cuda()
            d = torch.from_numpy(flat).cuda()
            ll = torch.empty((NP, B), device="cuda")
            streams = [torch.cuda.Stream() for _ in range(2)]
            torch.cuda.synchronize()
            check(lib.pcm_set_stream(forest.handle, streams[0].cuda_stream))
            check(lib.pcm_set_stream(top.handle, streams[1].cuda_stream))

            def step():
                check(lib.pcm_flows(forest.handle, d.data_ptr(), d.stride(0), d.stride(1), None, B, 0.0, dmask.data_ptr(),
                                    ll.data_ptr()))
                check(lib.pcm_em_update(forest.handle, 0.1, 0.9))
                check(lib.pcm_em_step(top.handle, dtop.data_ptr(), dtop.stride(0), dtop.stride(1), None, B, 0.0, 0.1, 0.9,
                                      ll_top.data_ptr()))
            how = "one forest handle"
        else:
            circs, datas, masks = [], [], []
            for p in range(NP):
                c = P.multihead_hclt_from_clt(parents[p], C, K, H)
                c.set_params(*params[p])                                     # heads stay uniform
                circs.append(c)
                datas.append(torch.from_numpy(np.ascontiguousarray(flat[:, pvars[p]])).cuda())
                m = np.zeros((H, B), np.float32)
                m[cluster[:, p], np.arange(B)] = 1.0
                masks.append(torch.from_numpy(m).cuda())
            lls = [torch.empty(B, device="cuda") for _ in range(NP)]
            streams = [torch.cuda.Stream() for _ in range(NS)]
            torch.cuda.synchronize()
            for i, c in enumerate(circs):
                check(lib.pcm_set_stream(c.handle, streams[i % NS].cuda_stream))
            check(lib.pcm_set_stream(top.handle, streams[0].cuda_stream))

            def step():
                for c, d, hm, ll in zip(circs, datas, masks, lls):
                    check(lib.pcm_flows(c.handle, d.data_ptr(), d.stride(0), d.stride(1), None, B, 0.0, hm.data_ptr(),
                                        ll.data_ptr()))
                    check(lib.pcm_em_update(c.handle, 0.1, 0.9))
                check(lib.pcm_em_step(top.handle, dtop.data_ptr(), dtop.stride(0), dtop.stride(1), None, B, 0.0, 0.1, 0.9,
                                      ll_top.data_ptr()))
            how = "%d handles on %d streams" % (NP, NS)
        dt = _timed(torch, step, args.steps, args.warmup)
        algo = sum(algorithmic_bytes(n, V, K, C, B)["step"] + 2 * 4 * H * B for n in n_int) \
            + algorithmic_bytes(top.size("inner_tree_nodes"), NP, 64, H, B)["step"]
        out.update(metric="images/sec fwd+bwd+EM, 12288-variable patch-clustered circuit: 64 patch circuits (192 vars, K=32, "
                          "128 heads; %s) + top HCLT (64 vars, K=64)" % how,
                   value=B / dt, unit="examples/s",
                   config={"workload": args.workload, "patch_circuits": NP, "num_vars": NP * V, "hidden": K,
                           "top_hidden": 64, "categories": C, "heads": H, "batch": B})
    elif args.workload == "c4_top_soft":
        # the top-level circuit of C4: 64 patch variables, 128 cluster categories, K = 64, trained on soft evidence
        V, K, C, B = 64, 64, 128, 1024
        data = workloads.grf_images(B, 8, 8, 1, 3.0, 0.8, seed=1005)
        parent = workloads.chow_liu_parent(data)
        theta, leaf = workloads.init_params(parent, K, C, 1105, kind="dirichlet")
        bpc = P.hclt_from_clt(parent, C, K)
        bpc.set_params(theta, leaf)
        ev = torch.from_numpy((rng.normal(-600, 30, (B, V, 1)) + rng.gumbel(0, 8, (B, V, C))).astype(np.float32)).cuda()
        ll = torch.empty(B, device="cuda")

        def step():
            check(lib.pcm_flows_soft(bpc.handle, ev.data_ptr(), ev.stride(0), ev.stride(1), ev.stride(2), None, B, 0.0, None,
                                     ll.data_ptr()))
            check(lib.pcm_em_update(bpc.handle, 0.1, 0.9))
        dt = _timed(torch, step, args.steps, args.warmup)
        nn, ne = bpc.num_nodes(), bpc.num_edges()
        # block form: the step's six K-vectors per tree node and example, the evidence read going up and down, the
        # per-example value table written once and read twice (up, down) and once more for the flows
        algo = algorithmic_bytes(bpc.size("inner_tree_nodes"), V, K, C, B)["step"] + 2 * 4 * B * V * C + 4 * 4 * B * V * K
        out.update(metric="examples/sec fwd+bwd+EM on soft evidence, 64-var HCLT K=64, 128 categories (block engine)",
                   value=B / dt, unit="examples/s",
                   config={"workload": args.workload, "num_vars": V, "hidden": K, "categories": C, "batch": B,
                           "nodes": nn, "edges": ne})
    elif args.workload == "hbm_stream_mix":
        # What the device's memory gives a kernel that only streams (pcm_stream_probe: 16 bytes per lane and
        # access, non-temporal, like the walks' tile traffic), per mix of reads and writes.  A "step" is one launch
        # of the backward walk's mix, 4 reads : 3 writes; the other mixes are listed beside it.
        lanes = 20 << 20                                    # 336 MB per stream
        src = torch.zeros(6 * lanes * 4, dtype=torch.float32, device="cuda")
        dst = torch.empty(3 * lanes * 4, dtype=torch.float32, device="cuda")
        stream = torch.cuda.current_stream().cuda_stream
        rates = {}
        for name, (r, w) in {"read_only": (1, 0), "write_only": (0, 1), "1r_1w": (1, 1), "backward_4r_3w": (4, 3),
                             "forward_1r_3w": (1, 3), "statistics_6r_1w": (6, 1)}.items():
            best = 0.0
            for grid in (1024, 2048, 8192):
                t = _timed(torch, lambda: check(lib.pcm_stream_probe(src.data_ptr(), dst.data_ptr(), lanes, r, w, grid, stream)),
                           max(3, args.steps // 5), 2)
                best = max(best, lanes * 16.0 * (r + w) / t / 1e9)
            rates[name] = best
        dt = _timed(torch, lambda: check(lib.pcm_stream_probe(src.data_ptr(), dst.data_ptr(), lanes, 4, 3, 2048, stream)),
                    args.steps, args.warmup)
        algo = lanes * 16.0 * 7
        out["dtype"] = "bytes"
        out.update(metric="GB/s of a plain streaming kernel, 4 reads : 3 writes of 16 B per lane, non-temporal",
                   value=algo / dt / 1e9, unit="GB/s",
                   config={"workload": args.workload, "bytes_per_stream": lanes * 16, "grid": 2048, "threads": 256},
                   mixes_gbs=rates)
    elif args.workload == "chow_liu_c3":
        cfg = workloads.make_config("c3_hclt3072_k32")
        V, C, B = cfg["V"], cfg["C"], cfg["B"]
        d = torch.from_numpy(cfg["data"]).cuda()
        P.pairwise_MI(d[:, :64], C, 0.1)
        t_mi = _timed(torch, lambda: P.pairwise_MI(d, C, 0.1), max(1, args.steps // 4), 1)
        mi = P.pairwise_MI(d, C, 0.1).cpu().numpy()
        t0 = time.perf_counter()
        parent = P.chow_liu_tree(mi)
        t_tree = time.perf_counter() - t0
        pairs = V * (V + 1) // 2
        dt = t_mi
        algo = pairs * 2 * B                                            # two rows of categories per pair (L2-served)
        note = "bytes requested: two rows of categories per pair of variables, served by L2; not HBM traffic"
        out["dtype"] = "u16 counts, f64 sums"
        out.update(metric="variable pairs/sec, pairwise mutual information of 4096 x 3072 uint8 data, 256 categories",
                   value=pairs / t_mi, unit="pairs/s",
                   config={"workload": args.workload, "num_vars": V, "categories": C, "examples": B},
                   structure_ms={"pairwise_mi": t_mi * 1e3, "spanning_tree_host": t_tree * 1e3},
                   tree={"depth": workloads.tree_stats(parent)["depth"]})
    else:
        print(f"unknown workload {args.workload}", file=sys.stderr)
        sys.exit(2)
    out["ms_per_step"] = dt * 1e3
    ach = algo / dt / 1e9
    out["roofline"] = {"bound": "hbm", "kernel": "whole step", "achieved": ach, "peak": HBM_PEAK_GBS,
                       "unit": "GB/s", "frac": ach / HBM_PEAK_GBS, "traffic": None}
    if note:
        out["roofline"]["note"] = note
        if note is REQUESTED_NOTE:   # a count of requests, most of them served by caches: no fraction of the HBM rate
            out["roofline"]["frac"] = None
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # the first ten or so steps of a fresh process run 3 % slower than the steady state (fresh pages of the
    # tile arrays, clocks): the default warm-up covers them
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c3_hclt3072_k32")
    ap.add_argument("--tree", choices=("chow_liu", "gaussian"), default="chow_liu",
                    help="chow_liu: learned by the library from 32768 training images; gaussian: host stand-in")
    ap.add_argument("--cpu-sample", type=int, default=4096)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--constant-categories", action="store_true",
                    help="ablation for the byte counters: every example shows category 0 everywhere after the tree is "
                         "built, so each leaf table is read at one row (what the leaf rows cost in fetches)")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MiB",
                    help="also launch one plain device copy of this many MiB before the timed region "
                         "(a known-size kernel to scale hardware byte counters against)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    import pcmi355
    from pcmi355 import workloads
    from pcmi355._lib import lib, check

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    if args.workload not in workloads.CONFIGS:
        return secondary(args)

    # the tree is learned as the reference learns it: pairwise mutual information of a training set and its
    # maximum spanning tree, both by the library (pcm_pairwise_mi, pcm_chow_liu_tree)
    cfg = workloads.make_config(args.workload, tree=args.tree)
    stats = workloads.tree_stats(cfg["parent"])
    V, K, C, B = cfg["V"], cfg["K"], cfg["C"], cfg["B"]
    bpc = pcmi355.hclt_from_clt(cfg["parent"], C, K)
    bpc.set_params(cfg["theta"], cfg["leaf"])
    data = torch.from_numpy(cfg["data"]).cuda()
    if args.constant_categories:
        data.zero_()
    ll = torch.empty(B, dtype=torch.float32, device="cuda")

    def step():
        check(lib.pcm_em_step(bpc.handle, data.data_ptr(), data.stride(0), data.stride(1), None, B, 0.0, 0.1, 0.9,
                              ll.data_ptr()))

    if args.calibrate_copy:
        src = torch.full((args.calibrate_copy << 20,), 7, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        step()
    # A timed dispatch costs a few microseconds, so the timed steps carry events on the dominant kernel only;
    # which one that is comes from twenty steps with all three timed, before the clock starts, and is confirmed
    # afterwards: the two longest kernels are within a few per cent of each other.
    bpc.set_timing(1)
    for _ in range(20):
        step()
    probe_ms = bpc.get_timing()
    dominant = max(probe_ms, key=probe_ms.get)
    bpc.set_timing(PHASE_MASK[dominant])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    dominant_ms = bpc.get_timing()[dominant]   # mean over the timed steps, events on the kernel's own dispatch
    bpc.set_timing(1)
    for _ in range(20):                        # the other two kernels, for the record: twenty further steps
        step()
    kernel_ms = bpc.get_timing()
    kernel_ms[dominant] = dominant_ms
    longest = max(kernel_ms, key=kernel_ms.get)
    if longest != dominant:
        # the probe picked the second-longest kernel: the longest one is timed alone over as many steps as the
        # timed region had (same state of the device, clock not running) and is the one reported
        bpc.set_timing(PHASE_MASK[longest])
        for _ in range(args.steps):
            step()
        kernel_ms[longest] = bpc.get_timing()[longest]
        if kernel_ms[longest] >= kernel_ms[dominant]:
            dominant = longest
    bpc.set_timing(0)
    ll_first = ll[:args.cpu_sample].cpu().numpy()

    ab = algorithmic_bytes(stats["n_inner"], V, K, C, B)
    achieved = ab[dominant] / (kernel_ms[dominant] * 1e-3) / 1e9
    ms_per_step = dt / args.steps * 1e3
    out = {
        "metric": "examples/sec fwd+bwd+EM, %d-var HCLT K=%d; %% of HBM/MFMA roofline" % (V, K),
        "value": B * args.steps / dt,
        "unit": "examples/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": args.workload, "num_vars": V, "hidden": K, "categories": C, "batch": B,
                   "tree": args.tree, "tree_inner_nodes": stats["n_inner"], "tree_depth": stats["depth"],
                   "tree_max_children": stats["max_children"]},
        "roofline": {"bound": "hbm", "kernel": KERNEL_NAMES[dominant] % K, "achieved": achieved,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "traffic": measured_traffic(args.workload, dominant)},
        "kernels_ms": kernel_ms,
        "step_roofline_frac": ab["step"] / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
    }
    if not args.no_cpu:
        # LL after `warmup + steps` parameter updates differs from the oracle's first step, so
        # the baseline is only timed here; parity lives in tests/.
        cb, _ = cpu_baseline(cfg, min(args.cpu_sample, B))
        out["cpu_baseline"] = cb
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
