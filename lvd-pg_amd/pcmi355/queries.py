"""Queries and learning loops, named after the reference functions they replace."""
import numpy as np
import torch

from ._lib import lib, check, np_ptr, c_i64


def _dev_ptr(t):
    return None if t is None else t.data_ptr()


def _is_soft(data):
    """The reference dispatches on `data isa CuArray{Float32,3}`: [examples, variables, categories] log-evidence."""
    return isinstance(data, torch.Tensor) and data.dim() == 3


def _check_data(bpc, data):
    if _is_soft(data):
        if not (data.is_cuda and data.dtype == torch.float32):
            raise ValueError("soft evidence must be a 3-D float32 tensor on the GPU (examples x variables x categories)")
        if data.shape[2] != bpc.size("categories"):
            raise ValueError(f"evidence has {data.shape[2]} categories, circuit has {bpc.size('categories')}")
    elif not (isinstance(data, torch.Tensor) and data.is_cuda and data.dtype == torch.uint8 and data.dim() == 2):
        raise ValueError("data must be a 2-D uint8 tensor on the GPU (examples x variables)")
    nv = bpc.size("variables")
    if data.shape[1] != nv:
        raise ValueError(f"data has {data.shape[1]} variables, circuit has {nv}")


def _forward(bpc, data, d_ptr, i_ptr, b, out_ptr):
    if _is_soft(data):
        check(lib.pcm_loglikelihoods_soft(bpc.handle, d_ptr, data.stride(0), data.stride(1), data.stride(2), i_ptr, b, out_ptr))
    else:
        check(lib.pcm_loglikelihoods(bpc.handle, d_ptr, data.stride(0), data.stride(1), i_ptr, b, out_ptr))


def _flows(bpc, data, i_ptr, b, rate, hm_ptr, ll_ptr):
    if _is_soft(data):
        check(lib.pcm_flows_soft(bpc.handle, data.data_ptr(), data.stride(0), data.stride(1), data.stride(2), i_ptr, b,
                                 float(rate), hm_ptr, ll_ptr))
    else:
        check(lib.pcm_flows(bpc.handle, data.data_ptr(), data.stride(0), data.stride(1), i_ptr, b, float(rate), hm_ptr, ll_ptr))


def _ids(example_ids, device):
    if example_ids is None:
        return None
    if isinstance(example_ids, torch.Tensor):
        return example_ids.to(device=device, dtype=torch.int32).contiguous()
    return torch.as_tensor(np.asarray(example_ids), dtype=torch.int32, device=device)


def loglikelihoods(bpc, data, batch_size=None, example_ids=None):
    """`loglikelihoods(bpc, data; batch_size)` / `loglikelihoods_probcat`
    (src/regularization/reg_likelihood.jl:139-162): per-example log-likelihoods as a device
    vector.  A multi-head circuit returns [num_examples, num_heads]
    (src-jl/multi_head_pc/likelihood.jl:37-71 with head_mask = nothing).  A 3-D float32 `data`
    [examples, variables, categories] is soft evidence (reg_likelihood.jl:51-91)."""
    _check_data(bpc, data)
    ids = _ids(example_ids, data.device)
    n = data.shape[0] if ids is None else len(ids)
    heads = getattr(bpc, "num_heads", 0)
    if n == 0:                                  # no examples: an empty result, no launch
        return torch.empty((0, heads) if heads else (0,), dtype=torch.float32, device=data.device)
    batch_size = n if batch_size is None else batch_size
    out = torch.empty((max(heads, 1), n), dtype=torch.float32, device=data.device)
    for s in range(0, n, batch_size):
        b = min(batch_size, n - s)
        if ids is None:
            d_ptr, i_ptr = data[s:s + b].data_ptr(), None
        else:
            d_ptr, i_ptr = data.data_ptr(), ids[s:s + b].data_ptr()
        if heads:
            tmp = torch.empty((heads, b), dtype=torch.float32, device=data.device)
            _forward(bpc, data, d_ptr, i_ptr, b, tmp.data_ptr())
            out[:, s:s + b] = tmp
        else:
            _forward(bpc, data, d_ptr, i_ptr, b, out[0, s:s + b].data_ptr())
    return out.t().contiguous() if heads else out[0]


def multihead_loglikelihoods(mhbpc, data, head_mask, batch_size=None, example_ids=None):
    """`loglikelihoods(mhbpc, data, head_mask; batch_size)`
    (src-jl/multi_head_pc/likelihood.jl:37-71) with a head mask [num_examples, num_heads]:
    logsumexp_h(ll_h + log mask_h) - log sum_h mask_h (:3-12), from the per-head values."""
    per_head = loglikelihoods(mhbpc, data, batch_size=batch_size, example_ids=example_ids)
    hm = head_mask.to(device=data.device, dtype=torch.float32)
    if example_ids is not None:
        hm = hm[_ids(example_ids, data.device).long()]
    return torch.logsumexp(per_head + torch.log(hm), dim=1) - torch.log(hm.sum(dim=1))


def loglikelihood(bpc, data, weights=None, batch_size=None, head_mask=None):
    """`loglikelihood_probcat(bpc, data, weights; batch_size)` (src/regularization/reg_likelihood.jl:164-173) and
    `weighted_ll` (src/regularization/reg_em.jl:191-197): the mean of the per-example log-likelihoods, weighted by
    `weights` (one per example) when given: sum(ll * w) / sum(w).  With `head_mask` the per-example values are the
    multi-head mixture's (`multihead_loglikelihoods`).  Returns a Python float; the sum runs in float64 on the device."""
    if head_mask is not None:
        lls = multihead_loglikelihoods(bpc, data, head_mask, batch_size=batch_size)
    else:
        lls = loglikelihoods(bpc, data, batch_size=batch_size)
    if lls.dim() != 1:
        raise ValueError("a multi-head circuit needs a head_mask to have one log-likelihood per example")
    if weights is None:
        return float(lls.sum(dtype=torch.float64).item()) / max(lls.numel(), 1)
    w = torch.as_tensor(weights).to(device=lls.device, dtype=torch.float64)
    if w.shape != lls.shape:
        raise ValueError(f"{w.numel()} weights for {lls.numel()} examples")
    return float(((lls.double() * w).sum() / w.sum()).item())


loglikelihoods_probcat = loglikelihoods        # reg_likelihood.jl:139-162: the same pass, the reference's other name
loglikelihood_probcat = loglikelihood          # reg_likelihood.jl:164-173


def weighted_ll(bpc, data, weights=None, batch_size=None, head_mask=None):
    """`weighted_ll` (src/regularization/reg_em.jl:191-197): without weights the per-example log-likelihoods (a
    device vector, as `loglikelihoods_probcat` returns them), with weights the scalar sum(ll * w) / sum(w).  With
    `head_mask` the per-example values are the multi-head mixture's."""
    if weights is None:
        if head_mask is not None:
            return multihead_loglikelihoods(bpc, data, head_mask, batch_size=batch_size)
        return loglikelihoods(bpc, data, batch_size=batch_size)
    return loglikelihood(bpc, data, weights, batch_size=batch_size, head_mask=head_mask)


def _check_weights(weights, n, device):
    """Per-example weights as a float32 device vector: one per example, finite and not negative (a negative
    weight would give edge and leaf statistics of different signs, a non-finite one has no fixed-point scale)."""
    w = torch.as_tensor(weights).to(device=device, dtype=torch.float32)
    if w.shape != (n,):
        raise ValueError(f"weights is {tuple(w.shape)}, the data has {n} examples")   # reg_em.jl:220
    if not bool((torch.isfinite(w) & (w >= 0)).all()):
        raise ValueError("weights must be finite and >= 0")
    return w


def probs_flows_circuit(bpc, data, example_ids=None, rate=0.0, head_mask=None, weights=None):
    """`probs_flows_circuit` (src/queries/flow.jl:228-234) /
    `probs_flows_circuit_with_reg` with soft_reg = 0 (src/regularization/reg_flow.jl:276-282):
    forward, backward and leaf flows for one batch; the aggregates stay in the circuit.
    Returns the batch's log-likelihoods (`mars[:, end]`).  `weights` (one per example of `data`) multiply the
    examples' edge and leaf flows (reg_flow.jl:38-39,190-191), see `mini_batch_em_with_reg`."""
    _check_data(bpc, data)
    ids = _ids(example_ids, data.device)
    b = data.shape[0] if ids is None else len(ids)
    ll = torch.empty(b, dtype=torch.float32, device=data.device)
    hm = None
    if head_mask is not None:
        hm = head_mask.to(device=data.device, dtype=torch.float32)
        if ids is not None:
            hm = hm[ids.long()]
    if weights is not None:
        w = _check_weights(weights, data.shape[0], data.device)
        if ids is not None:
            w = w[ids.long()]
        hm = w[:, None] if hm is None else hm * w[:, None]
    if hm is not None:
        hm = hm.t().contiguous()   # [heads (or 1), batch]
    _flows(bpc, data, _dev_ptr(ids), b, rate, _dev_ptr(hm), ll.data_ptr())
    return ll


def forest_loglikelihoods(forest, data, example_ids=None):
    """Per-head log-likelihoods of every tree of a forest handle for one batch, [trees, heads, examples]: what
    `loglikelihoods(mhbpc, data)` (src-jl/multi_head_pc/likelihood.jl:37-71) gives per patch circuit, transposed."""
    _check_data(forest, data)
    ids = _ids(example_ids, data.device)
    b = data.shape[0] if ids is None else len(ids)
    out = torch.empty((forest.size("trees"), forest.num_heads, b), dtype=torch.float32, device=data.device)
    if b:
        _forward(forest, data, data.data_ptr(), _dev_ptr(ids), b, out.data_ptr())
    return out


def forest_flows(forest, data, head_mask, example_ids=None, rate=0.0):
    """`probs_flows_circuit` of every tree of a forest handle for one batch.  head_mask: [trees, heads, examples of
    the batch] (src-jl/multi_head_pc/flow.jl:141-176 per tree); returns the mask-weighted log-likelihoods
    [trees, examples]."""
    _check_data(forest, data)
    ids = _ids(example_ids, data.device)
    b = data.shape[0] if ids is None else len(ids)
    T, Hn = forest.size("trees"), forest.num_heads
    hm = head_mask.to(device=data.device, dtype=torch.float32).contiguous()
    if tuple(hm.shape) != (T, Hn, b):
        raise ValueError(f"head_mask is {tuple(hm.shape)}, the forest needs {(T, Hn, b)}")
    ll = torch.empty((T, b), dtype=torch.float32, device=data.device)
    _flows(forest, data, _dev_ptr(ids), b, rate, hm.data_ptr(), ll.data_ptr())
    return ll


def soft_reg_evidence(rows, num_cats, soft_reg, soft_reg_width):
    """The categorical batch `rows` [B, V] (uint8) as the log-evidence [B, V, C] under which a leaf's value is
    the reference's `soft_loglikelihood` (src/regularization/reg_likelihood.jl:4-14):
    log((1 - soft_reg) * p[x] + soft_reg * mean(p[c] for c in the window)), the window being
    c_start = max(0, x - width ÷ 2) .. min(c_start + width - 1, C - 1)."""
    x = rows.long().unsqueeze(-1)
    c = torch.arange(num_cats, device=rows.device).view(1, 1, -1)
    c_start = (x - int(soft_reg_width) // 2).clamp_(min=0)
    c_end = (c_start + int(soft_reg_width) - 1).clamp_(max=num_cats - 1)
    w = ((c >= c_start) & (c <= c_end)).float() * (float(soft_reg) / (c_end - c_start + 1).float())
    w += (c == x).float() * (1.0 - float(soft_reg))
    return torch.log(w)


def mini_batch_em_with_reg(bpc, data, num_epochs, *, batch_size, pseudocount, soft_reg=0.0, soft_reg_width=1,
                           ent_reg=0.0, param_inertia, param_inertia_end=None, flow_memory=0.0,
                           shuffle="each_epoch", verbose=False, generator=None, head_mask=None, eval_dataset=None,
                           eval_interval=0, weights=None, eval_weights=None, init_clear_mem=True, soft_flow="derivative",
                           soft_reg_route=None):
    """`mini_batch_em_with_reg` (src/regularization/reg_em.jl:208-336).  Returns the list
    of per-epoch mean log-likelihoods.  ent_reg must be 0 (the reference's entropy regulariser is
    commented out at :294-296).  `data` may be 3-D float32 soft evidence, as for the top-level circuits of
    exps/LVD_for_imagenet/src/train_PG_top_level_pcs.jl.  With `verbose`, every `eval_interval` epochs the
    mean log-likelihood of `eval_dataset` is printed beside the training one (:308-327).

    `weights` (one per example of `data`, reg_em.jl:212,220) multiply an example's edge and leaf flows
    (reg_flow.jl:38-39,190-191); flows being linear in the flow an example starts with, they go in as that
    starting flow: a factor of the head mask for multi-head circuits, a one-row mask for single-root circuits.  The returned
    training likelihoods are unweighted as in the reference (:302); `eval_weights` weight the mean of the
    evaluation set (`weighted_ll`, :191-196).  `init_clear_mem = False` (src-jl/multi_head_pc/em.jl:6,28-31) keeps
    the flows the circuit holds from an earlier call as the flow memory of the first batch; the circuit owns its
    accumulators, so this is the reference's `edge_aggr_mem` given and not cleared.

    soft_reg > 0 on categorical data (reg_likelihood.jl:4-14, reg_flow.jl:3-22).  HCLT handles on the block kernels
    smooth inside the kernels (`pcm_set_soft_reg`: the leaves' smoothed values are a table of the shape of the leaf
    table, the walks run on the categories as they are); every other circuit has each batch turned into the soft
    evidence that gives the leaves the same value (`soft_reg_evidence`) and runs through the soft-evidence kernels
    (`soft_reg_route` = "kernels" / "evidence" insists on one of the two).  Likelihoods and inner flows are the
    reference's either way.  `soft_flow`: "derivative" shares a leaf's flow out as (1 - s) p[x] / base for the observed
    category and s / n * p[c] / base over the window -- the derivative of the smoothed value, the form of
    `soft_flow_params` (src/nodes/fixable_categorical_dist.jl:141-160); "as_written" as `soft_flow` itself computes it
    (reg_flow.jl:12-17), with log-probabilities where these probabilities stand: what the reference's own runs with
    soft_reg > 0 accumulate.  "as_written" needs the kernel route."""
    if ent_reg != 0.0:
        raise NotImplementedError("ent_reg other than 0 is not supported (commented out in the reference)")
    _check_data(bpc, data)
    smooth = soft_reg != 0.0 and not _is_soft(data)
    if smooth and not 0.0 < soft_reg < 1.0:
        raise ValueError("soft_reg must lie in [0, 1)")
    if soft_flow not in ("derivative", "as_written"):
        raise ValueError("soft_flow is 'derivative' or 'as_written'")
    in_kernels = False
    if smooth and soft_reg_route != "evidence":
        rc = lib.pcm_set_soft_reg(bpc.handle, float(soft_reg), int(soft_reg_width), int(soft_flow == "as_written"))
        in_kernels = rc == 0
        if not in_kernels and (soft_reg_route == "kernels" or soft_flow == "as_written"):
            check(rc)
    if smooth and not in_kernels and soft_flow == "as_written":
        raise NotImplementedError("soft_flow = 'as_written' needs the kernel route (an HCLT handle on the block kernels)")
    try:
        return _em_loop(bpc, data, num_epochs, batch_size, pseudocount, soft_reg, soft_reg_width, param_inertia,
                        param_inertia_end, flow_memory, shuffle, verbose, generator, head_mask, eval_dataset, eval_interval,
                        weights, eval_weights, init_clear_mem, smooth and not in_kernels)
    finally:
        if in_kernels:
            check(lib.pcm_set_soft_reg(bpc.handle, 0.0, 1, 0))


def _em_loop(bpc, data, num_epochs, batch_size, pseudocount, soft_reg, soft_reg_width, param_inertia, param_inertia_end,
             flow_memory, shuffle, verbose, generator, head_mask, eval_dataset, eval_interval, weights, eval_weights,
             init_clear_mem, smooth):
    """The batch loop of `mini_batch_em_with_reg` (src/regularization/reg_em.jl:236-336); `smooth`: soft_reg through
    the soft-evidence entry points."""
    n = data.shape[0]
    if batch_size > n:
        raise ValueError("batch_size must not exceed the number of examples")   # reg_em.jl:219
    num_batches = n // batch_size   # drop last incomplete batch (:217)
    if param_inertia_end is None:
        param_inertia_end = param_inertia
    d_inertia = (param_inertia_end - param_inertia) / num_epochs
    perm = torch.arange(n, dtype=torch.int32, device=data.device)

    def do_shuffle():
        nonlocal perm
        perm = torch.randperm(n, generator=generator).to(device=data.device, dtype=torch.int32)

    if shuffle == "once":
        do_shuffle()
    lls = []
    ll = torch.empty(batch_size, dtype=torch.float32, device=data.device)
    hm_t = None if head_mask is None else head_mask.to(device=data.device, dtype=torch.float32)
    w_t = None
    if weights is not None:
        w_t = _check_weights(weights, n, data.device)

    def batch_mask(ids):
        # [heads (or 1), batch]: the head mask of the batch, times the examples' weights
        if hm_t is None and w_t is None:
            return None
        if hm_t is None:
            return w_t[ids.long()][None, :].contiguous()
        hm = hm_t[ids.long()]
        if w_t is not None:
            hm = hm * w_t[ids.long()][:, None]
        return hm.t().contiguous()
    fresh = bool(init_clear_mem)   # the reference clears edge_aggr and the input nodes' flows before its loop (:243-244)
    for _ in range(num_epochs):
        if shuffle == "each_epoch":
            do_shuffle()
        acc = torch.zeros((), dtype=torch.float64, device=data.device)
        for bi in range(num_batches):
            if shuffle == "each_batch":
                do_shuffle()
            ids = perm[bi * batch_size:(bi + 1) * batch_size]
            rate = 0.0 if (flow_memory == 0 or fresh) else max(0.0, 1.0 - (batch_size + pseudocount) / flow_memory)
            fresh = False
            if smooth:
                ev = soft_reg_evidence(data[ids.long()], bpc.size("categories"), soft_reg, soft_reg_width)
                hm = batch_mask(ids)
                _flows(bpc, ev, None, batch_size, rate, _dev_ptr(hm), ll.data_ptr())
                check(lib.pcm_em_update(bpc.handle, float(pseudocount), float(param_inertia)))
            elif hm_t is None and w_t is None and not _is_soft(data):
                check(lib.pcm_em_step(bpc.handle, data.data_ptr(), data.stride(0), data.stride(1), ids.data_ptr(),
                                      batch_size, rate, float(pseudocount), float(param_inertia), ll.data_ptr()))
            else:
                hm = batch_mask(ids)
                _flows(bpc, data, ids.data_ptr(), batch_size, rate, _dev_ptr(hm), ll.data_ptr())
                check(lib.pcm_em_update(bpc.handle, float(pseudocount), float(param_inertia)))
            acc += ll.sum(dtype=torch.float64)
        lls.append(float(acc.item()) / batch_size / num_batches)
        param_inertia += d_inertia
        if verbose:
            epoch = len(lls)
            if eval_dataset is not None and eval_interval > 0 and epoch % eval_interval == 0 and hm_t is None:
                test_ll = loglikelihood(bpc, eval_dataset, eval_weights, batch_size=min(batch_size, eval_dataset.shape[0]))
                print(f"Mini-batch EM epoch {epoch}/{num_epochs}: train LL {lls[-1]} - test LL {test_ll}")
            else:
                print(f"Mini-batch EM epoch {epoch}/{num_epochs}; train LL {lls[-1]}")
    return lls


def mini_batch_em_beta(bpc, data, num_epochs, *, batch_size, pseudocount, soft_reg=0.0, soft_reg_width=1, param_inertia,
                       param_inertia_end=None, flow_memory=0.0, flow_memory_end=None, shuffle="each_epoch",
                       update_interval=1, fscale=1.0, verbose=False, generator=None, eval_dataset=None, eval_interval=0,
                       soft_flow="derivative"):
    """`mini_batch_em_beta` (src-jl/learning/em.jl:289-409): the EM loop whose statistics collect over
    `update_interval` batches before the parameters move, with a schedule for the flow memory as well as for the
    inertia.  As the source has it: the accumulators are cleared at the start of every epoch; at a batch with
    `batch_id % update_interval == 1` (1-based) they are cleared again (flow_memory = 0) or scaled by
    max(0, 1 - (batch_size + pseudocount) / flow_memory); every batch adds its flows; after a batch with
    `batch_id % update_interval == 0` the parameters are updated.  (With update_interval = 1 the first condition never
    holds, so the statistics of an epoch pile up while the parameters move after every batch -- kept as written.)
    `fscale` other than 1: the flows of the tempered posterior (`scaled_probs_flows_circuit`,
    src-jl/learning/flow.jl:120-373), set on the handle for the length of the loop (`pcm_set_flow_scale`; an HCLT handle
    runs them on its layered form).  soft_reg > 0 with fscale = 1 needs an HCLT handle on the block kernels
    (`pcm_set_soft_reg`); with fscale other than 1 the library turns every batch into the soft evidence that gives the
    leaves the smoothed values, with tempered flows above them and the leaf flows in their "derivative" form --
    `soft_flow = "as_written"` is the block kernels' and raises NotImplementedError there.
    Returns the per-epoch mean log-likelihoods."""
    if fscale != 1.0 and soft_reg != 0.0 and soft_flow == "as_written":
        raise NotImplementedError("soft_flow = 'as_written' together with fscale other than 1: that form of the leaf flows "
                                  "runs in the block kernels, the tempered flows on the layered engine")
    if not (fscale > 0 and np.isfinite(fscale)):
        raise ValueError("fscale must be positive and finite")
    _check_data(bpc, data)
    if pseudocount < 0 or not 0 <= param_inertia <= 1:
        raise ValueError("pseudocount >= 0 and 0 <= param_inertia <= 1")                        # em.jl:299-300
    param_inertia_end = param_inertia if param_inertia_end is None else param_inertia_end
    flow_memory_end = flow_memory if flow_memory_end is None else flow_memory_end
    if not param_inertia <= param_inertia_end <= 1 or not 0 <= flow_memory <= flow_memory_end:
        raise ValueError("param_inertia <= param_inertia_end <= 1 and 0 <= flow_memory <= flow_memory_end")   # :301-303
    if shuffle not in ("once", "each_epoch", "each_batch", "none"):
        raise ValueError("shuffle is once, each_epoch or each_batch")
    if update_interval < 1:
        raise ValueError("update_interval must be at least 1")
    n = data.shape[0]
    if batch_size > n:
        raise ValueError("batch_size must not exceed the number of examples")
    num_batches = n // batch_size
    smooth = soft_reg != 0.0
    if smooth and not 0.0 < soft_reg < 1.0:
        raise ValueError("soft_reg must lie in [0, 1)")
    if smooth:
        check(lib.pcm_set_soft_reg(bpc.handle, float(soft_reg), int(soft_reg_width), int(soft_flow == "as_written")))
    if fscale != 1.0:
        check(lib.pcm_set_flow_scale(bpc.handle, float(fscale)))
    perm = torch.arange(n, dtype=torch.int32, device=data.device)

    def do_shuffle():
        nonlocal perm
        perm = torch.randperm(n, generator=generator).to(device=data.device, dtype=torch.int32)

    d_inertia = (param_inertia_end - param_inertia) / num_epochs
    d_memory = (flow_memory_end - flow_memory) / num_epochs
    ll = torch.empty(batch_size, dtype=torch.float32, device=data.device)
    lls = []
    try:
        if shuffle == "once":
            do_shuffle()
        for epoch in range(1, num_epochs + 1):
            if shuffle == "each_epoch":
                do_shuffle()
            acc = torch.zeros((), dtype=torch.float64, device=data.device)
            cleared = True                                                                      # em.jl:344-345
            for batch_id in range(1, num_batches + 1):
                if shuffle == "each_batch":
                    do_shuffle()
                rate = 1.0
                if batch_id % update_interval == 1:                                             # :354-363
                    rate = 0.0 if flow_memory == 0 else max(0.0, 1.0 - (batch_size + pseudocount) / flow_memory)
                if cleared:
                    rate, cleared = 0.0, False
                ids = perm[(batch_id - 1) * batch_size:batch_id * batch_size]
                _flows(bpc, data, ids.data_ptr(), batch_size, rate, None, ll.data_ptr())
                acc += ll.sum(dtype=torch.float64)
                if batch_id % update_interval == 0:                                             # :373-379
                    check(lib.pcm_em_update(bpc.handle, float(pseudocount), float(param_inertia)))
            lls.append(float(acc.item()) / batch_size / num_batches)
            param_inertia += d_inertia
            flow_memory += d_memory
            if verbose:
                if eval_dataset is not None and eval_interval > 0 and epoch % eval_interval == 0:
                    test_ll = loglikelihood(bpc, eval_dataset, batch_size=min(batch_size, eval_dataset.shape[0]))
                    print(f"Mini-batch EM epoch {epoch}/{num_epochs}: train LL {lls[-1]} - test LL {test_ll}")
                else:
                    print(f"Mini-batch EM epoch {epoch}/{num_epochs}; train LL {lls[-1]}")
    finally:
        if smooth:
            check(lib.pcm_set_soft_reg(bpc.handle, 0.0, 1, 0))
        if fscale != 1.0:
            check(lib.pcm_set_flow_scale(bpc.handle, 1.0))
    return lls


def mini_batch_em(bpc, data, num_epochs, *, batch_size, pseudocount, param_inertia, param_inertia_end=None,
                  flow_memory=0.0, shuffle="each_epoch", **kw):
    """`PCs.mini_batch_em` as called by test/sgd/adam_tests.jl:20: the same loop without
    regularisers."""
    return mini_batch_em_with_reg(bpc, data, num_epochs, batch_size=batch_size, pseudocount=pseudocount,
                                  param_inertia=param_inertia, param_inertia_end=param_inertia_end,
                                  flow_memory=flow_memory, shuffle=shuffle, **kw)


def mini_batch_em_for_multihead_pc(mhbpc, data, head_mask, num_epochs, **kw):
    """`mini_batch_em_for_multihead_pc` (src-jl/multi_head_pc/em.jl:1-99)."""
    return mini_batch_em_with_reg(mhbpc, data, num_epochs, head_mask=head_mask, **kw)


def mini_batch_em_for_forest(forest, data, head_masks, num_epochs, *, batch_size, pseudocount, param_inertia,
                             param_inertia_end=None, flow_memory=0.0, shuffle="each_epoch", generator=None,
                             weights=None):
    """The loop over patch circuits of exps/progressive_growing/parallel_PG.jl:214-225 -- one
    `mini_batch_em_for_multihead_pc` (src-jl/multi_head_pc/em.jl:1-99) per circuit -- as one loop over a forest handle:
    every batch is one `pcm_flows` + `pcm_em_update` for all trees, with the batch order, inertia schedule and flow
    memory of `mini_batch_em_with_reg`.  head_masks: [trees, examples, heads], a tree's slice being the `head_mask`
    the reference passes for that circuit; `weights` (one per example, em.jl:5,20) multiply an example's flows in
    every tree, as a factor of its masks.  Returns the per-epoch mean log-likelihoods, [epochs, trees]."""
    _check_data(forest, data)
    n, T = data.shape[0], forest.size("trees")
    if batch_size > n:
        raise ValueError("batch_size must not exceed the number of examples")
    hm_t = head_masks.to(device=data.device, dtype=torch.float32)
    if tuple(hm_t.shape) != (T, n, forest.num_heads):
        raise ValueError(f"head_masks is {tuple(hm_t.shape)}, the forest needs {(T, n, forest.num_heads)}")
    if weights is not None:
        hm_t = hm_t * _check_weights(weights, n, data.device)[None, :, None]
    num_batches = n // batch_size
    if param_inertia_end is None:
        param_inertia_end = param_inertia
    d_inertia = (param_inertia_end - param_inertia) / num_epochs
    perm = torch.arange(n, dtype=torch.int32, device=data.device)

    def do_shuffle():
        nonlocal perm
        perm = torch.randperm(n, generator=generator).to(device=data.device, dtype=torch.int32)

    if shuffle == "once":
        do_shuffle()
    lls, fresh = [], True
    ll = torch.empty((T, batch_size), dtype=torch.float32, device=data.device)
    for _ in range(num_epochs):
        if shuffle == "each_epoch":
            do_shuffle()
        acc = torch.zeros(T, dtype=torch.float64, device=data.device)
        for bi in range(num_batches):
            if shuffle == "each_batch":
                do_shuffle()
            ids = perm[bi * batch_size:(bi + 1) * batch_size]
            rate = 0.0 if (flow_memory == 0 or fresh) else max(0.0, 1.0 - (batch_size + pseudocount) / flow_memory)
            fresh = False
            hm = hm_t[:, ids.long()].transpose(1, 2).contiguous()   # [trees, heads, batch]
            _flows(forest, data, ids.data_ptr(), batch_size, rate, hm.data_ptr(), ll.data_ptr())
            check(lib.pcm_em_update(forest.handle, float(pseudocount), float(param_inertia)))
            acc += ll.sum(dim=1, dtype=torch.float64)
        lls.append((acc / batch_size / num_batches).cpu().numpy())
        param_inertia += d_inertia
    return np.stack(lls)


def vectorize_parameters(bpc):
    """`vectorize_parameters(mbpc)` (src/misc.jl:33-40) -> host float32 vector."""
    out = np.empty(bpc.num_parameters(), np.float32)
    check(lib.pcm_vectorize_parameters(bpc.handle, np_ptr(out), c_i64(len(out))))
    return out


def update_parameters(bpc, params):
    """`update_parameters(mbpc, params)` (src/misc.jl:73-102)."""
    p = np.ascontiguousarray(params, np.float32)
    if len(p) != bpc.num_parameters():   # the reference asserts the same (:75)
        raise ValueError(f"{bpc.num_parameters()} != {len(p)}")
    check(lib.pcm_update_parameters(bpc.handle, np_ptr(p), c_i64(len(p))))


def _rows_on_device(x, n, what):
    """A parameter matrix [rows, n] as a float32 GPU tensor (host arrays are uploaded); returns
    (tensor, was_host)."""
    host = not isinstance(x, torch.Tensor)
    t = torch.as_tensor(np.ascontiguousarray(x, np.float32) if host else x)
    if t.dim() != 2 or t.shape[1] != n:
        raise ValueError(f"{what} must be [rows, {n}], got {tuple(t.shape)}")
    if t.dtype != torch.float32:
        t = t.float()
    return (t.cuda() if not t.is_cuda else t), host


def per_sample_normalized_flows(mbpc, data, *, batch_size=None, as_written=True, out=None):
    """`per_sample_normalized_flows(mbpc, data; batch_size)` (src/queries/flow.jl:417-464): for every example the
    vector, in parameter order, of its flows normalised per sum node and per input node --
    log(f / (g + 1e-8) + 1e-8) for a sum parameter (`map_flows_kernel`, :496-528) and log(f_c / sum_c f_c) for an
    input parameter (`map_input_flows_kernel`, :549-593).  The circuit's accumulators are not touched.  `data` is a
    uint8 GPU tensor or host array [examples, variables]; returns [examples, num_parameters] float32, a host array
    for host data (the reference returns `Array(normalized_flows)`), a GPU tensor otherwise or when `out` (a float32
    GPU tensor of that shape, any strides) is given.
    as_written: the input node's flow lands where `get_edge_flow` (src/nodes/fixable_categorical_dist.jl:162-176) puts
    it, which compares the 0-based category with the 1-based parameter index: category x fills the slot of category
    x - 1 and category 0 none (its node's entries are NaN).  False: the slot of the observed category."""
    host = not isinstance(data, torch.Tensor)
    d = torch.as_tensor(np.ascontiguousarray(data, np.uint8)).cuda() if host else data
    _check_data(mbpc, d)
    n, npar = d.shape[0], mbpc.num_parameters()
    if out is None:
        out = torch.empty((n, npar), dtype=torch.float32, device=d.device)
    elif tuple(out.shape) != (n, npar) or out.dtype != torch.float32 or not out.is_cuda:
        raise ValueError(f"out must be a float32 GPU tensor of shape {(n, npar)}")
    batch_size = n if batch_size is None else int(batch_size)
    for s in range(0, n, max(batch_size, 1)):
        part = d[s:s + batch_size]
        o = out[s:s + batch_size]
        check(lib.pcm_normalized_flows(mbpc.handle, part.data_ptr(), part.stride(0), part.stride(1), None, part.shape[0],
                                       int(bool(as_written)), o.data_ptr(), o.stride(0), o.stride(1)))
    return out.cpu().numpy() if host else out


def normalize_params(mbpc, params, *, undo=False):
    """`normalize_params(mbpc, params; undo)` (src/misc.jl:448-498) on a matrix [rows, num_parameters]: input
    entries -> exp(entry) / sum over the node (probabilities; undo: p > 0 -> log(p + 1e-6)), sum parameters ->
    logp - log(sum over the node of exp(logp)).  A GPU tensor is changed in place and returned; a host array comes
    back as a new host array (the reference returns `Array(params)`)."""
    p, host = _rows_on_device(params, mbpc.num_parameters(), "params")
    check(lib.pcm_normalize_params_rows(mbpc.handle, p.data_ptr(), p.stride(0), p.stride(1), p.shape[0], int(bool(undo))))
    return p.cpu().numpy() if host else p


def map_pc_parameters(mbpc1, mbpc2, params2, *, param_mapping, params1=None):
    """`map_pc_parameters(mbpc1, mbpc2, params1, params2; param_mapping)` (src/utils/map_params.jl:12-45, kernel
    :128-146): params1[:, ids1[i]] = params2[:, ids2[i]] for the matched parameter pairs `param_mapping = (ids1,
    ids2)`, 1-based as `compute_mbpc_mapping` (:47-126) gives them; unmatched columns of params1 keep what they
    held (zeros for a new matrix, as :7).  GPU tensors in and out."""
    ids1, ids2 = (torch.as_tensor(np.asarray(x, np.int64) - 1) for x in param_mapping)
    p2, _ = _rows_on_device(params2, mbpc2.num_parameters(), "params2")
    if params1 is None:
        params1 = torch.zeros((p2.shape[0], mbpc1.num_parameters()), dtype=torch.float32, device=p2.device)
    if ids1.numel() and (int(ids1.max()) >= params1.shape[1] or int(ids2.max()) >= p2.shape[1] or int(ids1.min()) < 0
                         or int(ids2.min()) < 0):
        raise ValueError("param_mapping names parameters the circuits do not have")
    params1[:, ids1.to(p2.device)] = p2[:, ids2.to(p2.device)]
    return params1


def kld(mbpc, params1, params2=None, *, norm_params=False):
    """`kld(mbpc, params1, params2; norm_params)` (src/queries/kld.jl:164-206): KL(row r of params1
    || row r of params2) for every row of the two [rows, num_parameters] matrices (host arrays
    or GPU tensors, any strides), all rows in one pass; returns `klds[:, end]` as a host vector
    (GPU tensor for GPU input).  With norm_params the leaf parameters are probabilities.
    Called with a second circuit instead, `kld(bpc_p, bpc_q)`, it takes the two circuits' own
    parameters as the single row and returns a float."""
    if params2 is None:
        out = np.zeros(1, np.float32)
        check(lib.pcm_kld(mbpc.handle, params1.handle, np_ptr(out)))
        return float(out[0])
    n = mbpc.num_parameters()
    p1, host = _rows_on_device(params1, n, "params1")
    p2, _ = _rows_on_device(params2, n, "params2")
    if p2.shape[0] == 1 and p1.shape[0] > 1:
        p2 = p2.expand(p1.shape[0], n).contiguous()
    if p2.shape != p1.shape or p2.stride() != p1.stride():
        p1, p2 = p1.contiguous(), p2.contiguous()
    if p1.shape != p2.shape:
        raise ValueError("params1 and params2 must have the same shape")
    out = torch.empty(p1.shape[0], dtype=torch.float32, device=p1.device)
    check(lib.pcm_kld_rows(mbpc.handle, p1.data_ptr(), p2.data_ptr(), p1.stride(0), p1.stride(1), p1.shape[0],
                           int(bool(norm_params)), out.data_ptr()))
    return out.cpu().numpy() if host else out


def kld_backward(mbpc, params1, params2=None, *, device=False, norm_params=False, grad_wrt_logparams=True):
    """`kld_backward(mbpc, params1, params2; norm_params, grad_wrt_logparams = true)`
    (src/queries/kld.jl:593-649) -> (grads1, grads2), matrices shaped like the parameter
    matrices, all rows in one pass.  Called with a second circuit instead it differentiates
    the single row of the two circuits' own parameters: host vectors, or with device=True GPU
    tensors (what adam_step takes)."""
    if not grad_wrt_logparams:
        raise NotImplementedError("grad_wrt_logparams = false: the reference's kernel for it is empty (kld.jl:322-331)")
    n = mbpc.num_parameters()
    if params2 is None:
        bpc_q = params1
        if device:
            g1 = torch.empty(n, dtype=torch.float32, device="cuda")
            g2 = torch.empty(n, dtype=torch.float32, device="cuda")
            check(lib.pcm_kld_backward_dev(mbpc.handle, bpc_q.handle, g1.data_ptr(), g2.data_ptr(), c_i64(n)))
            return g1, g2
        g1 = np.empty(n, np.float32)
        g2 = np.empty(n, np.float32)
        check(lib.pcm_kld_backward(mbpc.handle, bpc_q.handle, np_ptr(g1), np_ptr(g2), c_i64(n)))
        return g1, g2
    p1, host = _rows_on_device(params1, n, "params1")
    p2, _ = _rows_on_device(params2, n, "params2")
    if p2.shape[0] == 1 and p1.shape[0] > 1:
        p2 = p2.expand(p1.shape[0], n).contiguous()
    if p2.shape != p1.shape or p2.stride() != p1.stride():
        p1, p2 = p1.contiguous(), p2.contiguous()
    if p1.shape != p2.shape:
        raise ValueError("params1 and params2 must have the same shape")
    g1, g2 = torch.empty_strided(p1.shape, p1.stride(), dtype=torch.float32, device=p1.device), \
        torch.empty_strided(p1.shape, p1.stride(), dtype=torch.float32, device=p1.device)
    check(lib.pcm_kld_backward_rows(mbpc.handle, p1.data_ptr(), p2.data_ptr(), p1.stride(0), p1.stride(1), p1.shape[0],
                                    int(bool(norm_params)), g1.data_ptr(), g2.data_ptr(), None))
    return (g1.cpu().numpy(), g2.cpu().numpy()) if host else (g1, g2)


def gumbel_sample_rows(mbpc, params, *, temperature, noise=None, norm_params=False):
    """`gumbel_sample(mbpc, params, num_vars, par_buffer_size; temperature, no_gumbel, norm_params)`
    (src/queries/sample.jl:338-383) for a [rows, num_parameters] matrix: one relaxed top-down
    pass per row, all rows at once.  noise: [rows, num sum parameters] Gumbel draws (one per sum
    edge, as the reference draws them in its kernel, :45), or None for no_gumbel = true.
    Returns the soft assignment [rows, V, C] (host array for host input, else GPU tensor)."""
    n = mbpc.num_parameters()
    p, host = _rows_on_device(params, n, "params")
    ns = mbpc.num_inner_params()
    if noise is not None:
        noise, _ = _rows_on_device(noise, ns, "noise")
        noise = noise.contiguous()
        if noise.shape[0] != p.shape[0]:
            raise ValueError("noise must have one row per parameter row")
    out = torch.empty((p.shape[0], mbpc.size("variables"), mbpc.size("categories")), dtype=torch.float32, device=p.device)
    check(lib.pcm_gumbel_sample_rows(mbpc.handle, p.data_ptr(), p.stride(0), p.stride(1), p.shape[0], _dev_ptr(noise),
                                     float(temperature), int(bool(norm_params)), out.data_ptr()))
    return out.cpu().numpy() if host else out


def gumbel_sample_backward_rows(mbpc, params, out_grads, *, temperature, noise=None, norm_params=False,
                                grad_wrt_logparams=True):
    """`gumbel_sample_backward(mbpc, params, input_aggr_params, input_aggr_grads, temperature; norm_params,
    grad_wrt_logparams)` (src/queries/sample.jl:620-692): gradients of a loss with respect to every row of
    `params`, given its gradients `out_grads` [rows, V, C] with respect to the soft assignment that
    `gumbel_sample_rows` returned for the same params, noise and temperature.  Leaf entries are gradients
    per probability of the category, as the source writes them (:560-570).  Returns [rows, num_parameters]
    (host array for host input, else GPU tensor with the strides of `params`)."""
    n = mbpc.num_parameters()
    p, host = _rows_on_device(params, n, "params")
    rows = p.shape[0]
    if noise is not None:
        noise, _ = _rows_on_device(noise, mbpc.num_inner_params(), "noise")
        noise = noise.contiguous()
        if noise.shape[0] != rows:
            raise ValueError("noise must have one row per parameter row")
    og = torch.as_tensor(out_grads, dtype=torch.float32, device=p.device).contiguous()
    if tuple(og.shape) != (rows, mbpc.size("variables"), mbpc.size("categories")):
        raise ValueError("out_grads must be [rows, num_vars, num_cats]")
    g = torch.empty_strided(p.shape, p.stride(), dtype=torch.float32, device=p.device)
    check(lib.pcm_gumbel_sample_backward_rows(mbpc.handle, p.data_ptr(), p.stride(0), p.stride(1), rows, _dev_ptr(noise),
                                              float(temperature), int(bool(norm_params)), int(bool(grad_wrt_logparams)),
                                              og.data_ptr(), g.data_ptr()))
    return g.cpu().numpy() if host else g


def sample(bpc, node_noise, leaf_noise):
    """Gumbel-max samples from supplied noise (temperature -> 0 limit of `gumbel_sample`,
    src/queries/sample.jl:338-383).  node_noise [B, sample_noise_size], leaf_noise
    [B, V, C], float32 on the GPU.  Returns uint8 [B, V] on the GPU."""
    b = node_noise.shape[0]
    need = int(lib.pcm_sample_noise_size(bpc.handle))
    nv, nc = bpc.size("variables"), bpc.size("categories")
    if tuple(node_noise.shape) != (b, need) or tuple(leaf_noise.shape) != (b, nv, nc):
        raise ValueError(f"noise shapes must be ({b}, {need}) and ({b}, {nv}, {nc})")
    node_noise = node_noise.contiguous().float()
    leaf_noise = leaf_noise.contiguous().float()
    out = torch.empty((b, nv), dtype=torch.uint8, device=node_noise.device)
    check(lib.pcm_sample(bpc.handle, node_noise.data_ptr(), leaf_noise.data_ptr(), b, out.data_ptr()))
    return out


def gumbel_sample(bpc, num_samples, *, temperature, node_noise=None):
    """`gumbel_sample(mbpc, params, num_vars, par_buffer_size; temperature, no_gumbel)`
    (src/queries/sample.jl:338-383): relaxed top-down sampling.  node_noise
    [num_samples, sample_noise_size] float32 on the GPU, or None for no_gumbel = true.
    Returns the soft assignment [num_samples, V, C] (float32, GPU)."""
    nv, nc = bpc.size("variables"), bpc.size("categories")
    need = int(lib.pcm_sample_noise_size(bpc.handle))
    if node_noise is not None:
        if tuple(node_noise.shape) != (num_samples, need):
            raise ValueError(f"noise shape must be ({num_samples}, {need})")
        node_noise = node_noise.contiguous().float()
        dev = node_noise.device
    else:
        dev = torch.device("cuda")
    out = torch.empty((num_samples, nv, nc), dtype=torch.float32, device=dev)
    check(lib.pcm_sample_soft(bpc.handle, _dev_ptr(node_noise), float(temperature), int(num_samples), out.data_ptr()))
    return out


def adam_step(bpc, grad, params, m, v, *, lr, beta1=0.9, beta2=0.999, eps=1e-8, t=1):
    """One optimiser step of `adam` (src/sgd/adam.jl:318-325): moving averages, ascent
    update of the unnormalised sum parameters, per-node normalisation into the circuit."""
    check(lib.pcm_adam_step(bpc.handle, grad.data_ptr(), params.data_ptr(), m.data_ptr(), v.data_ptr(),
                            float(lr), float(beta1), float(beta2), float(eps), int(t)))


def flow_gradients(bpc, batch_size):
    """`edge_aggr ./= batch_size; compute_gradients(bpc, edge_aggr, node_aggr)` (src/sgd/adam.jl:310-311,
    :27-61) on the flows the circuit holds: the gradient of the mean log-likelihood with respect to the
    unnormalised sum log-parameters, a GPU vector in parameter order."""
    g = torch.empty(bpc.num_inner_params(), dtype=torch.float32, device="cuda")
    check(lib.pcm_flow_gradients(bpc.handle, int(batch_size), g.data_ptr()))
    return g


def adam(bpc, data, num_epochs, *, batch_size, lr, beta1=0.9, beta2=0.999, eps=1e-8, verbose=False, generator=None,
         shuffle=True, state=None):
    """`adam(bpc, data, num_epochs; batch_size, lr, beta1, beta2, eps)` (src/sgd/adam.jl:244-344): per batch the
    flows, the gradient from them, Adam on the unnormalised sum log-parameters with per-node renormalisation
    into the circuit, and the input nodes' Adam on an auxiliary copy of their parameters (which, as in the
    source, never flows back into the circuit).  Returns the per-epoch mean log-likelihoods.  `state`, if given,
    is a dict that receives the optimiser arrays (params, m, v, leaf_params, leaf_m, leaf_v, opt_count)."""
    _check_data(bpc, data)
    n = data.shape[0]
    if batch_size > n:
        raise ValueError("batch_size must not exceed the number of examples")    # adam.jl:258
    num_batches = n // batch_size
    dev = data.device
    ns, nl = bpc.num_inner_params(), bpc.num_input_params()
    pv = torch.from_numpy(vectorize_parameters(bpc)).to(dev)
    params = pv[:ns].clone()                  # copy_parameters_to_vec (:150-172)
    leaf_params = pv[ns:].clone()             # copy_input_parameters_to_heap (:174-203)
    m, v = torch.zeros_like(params), torch.zeros_like(params)
    leaf_m, leaf_v = torch.zeros_like(leaf_params), torch.zeros_like(leaf_params)
    ll = torch.empty(batch_size, dtype=torch.float32, device=dev)
    perm = torch.arange(n, dtype=torch.int32, device=dev)
    lls, opt_count = [], 0
    for epoch in range(num_epochs):
        if shuffle:
            perm = torch.randperm(n, generator=generator).to(device=dev, dtype=torch.int32)
        acc = torch.zeros((), dtype=torch.float64, device=dev)
        for bi in range(num_batches):
            opt_count += 1
            ids = perm[bi * batch_size:(bi + 1) * batch_size]
            _flows(bpc, data, ids.data_ptr(), batch_size, 0.0, None, ll.data_ptr())
            acc += ll.sum(dtype=torch.float64)
            check(lib.pcm_adam_flow_step(bpc.handle, batch_size, params.data_ptr(), m.data_ptr(), v.data_ptr(),
                                         leaf_params.data_ptr(), leaf_m.data_ptr(), leaf_v.data_ptr(), float(lr),
                                         float(beta1), float(beta2), float(eps), opt_count))
        lls.append(float(acc.item()) / batch_size / num_batches)
        if verbose:
            print(f"Adam epoch {epoch + 1}; train LL {lls[-1]}")
    if state is not None:
        state.update(params=params, m=m, v=v, leaf_params=leaf_params, leaf_m=leaf_m, leaf_v=leaf_v, opt_count=opt_count)
    return lls


def patch_level_evidence(mhbpcs, patches, batch_size=256):
    """The pseudo dataset of the top-level circuit
    (exps/LVD_for_imagenet/src/train_PG_top_level_pcs.jl:82-118): for every patch (a uint8
    device tensor [N, patch variables]) the per-head log-likelihoods of every multi-head patch
    circuit, heads of all circuits side by side.  Returns float32 [N, patches, heads in total],
    the soft-evidence input of `mini_batch_em_with_reg` / `loglikelihoods`."""
    mhbpcs = list(mhbpcs)
    total = sum(max(getattr(m, "num_heads", 0), 1) for m in mhbpcs)
    n = patches[0].shape[0]
    out = torch.empty((n, len(patches), total), dtype=torch.float32, device=patches[0].device)
    for p, x in enumerate(patches):
        if x.shape[0] != n:
            raise ValueError("every patch must hold the same examples")
        x = x.contiguous()
        h0 = 0
        for m in mhbpcs:
            ll = loglikelihoods(m, x, batch_size=min(batch_size, n))
            ll = ll if ll.dim() == 2 else ll[:, None]
            out[:, p, h0:h0 + ll.shape[1]] = ll
            h0 += ll.shape[1]
    return out
