# Host side of libpcmi355 in Julia: the reference's call signatures for the probabilistic-circuit hot path
# (VariationalJuice.jl; file:line citations below are relative to it) on top of the raw bindings of LibPCMI355.jl.
#
# No CUDA.jl, no AMDGPU.jl: device memory is a pointer from hipMalloc (through `ccall` into the HIP runtime the
# library itself links), wrapped in `DeviceArray`.  Anything else that can give a device address -- an
# AMDGPU.ROCArray, a buffer of the caller's own allocator -- goes through the same functions by defining
# `PCMI355.device_pointer(x)` for it.  Arrays are column-major as Julia holds them: element (example e,
# variable v) of a [N, V] matrix is at e + N*v, which the library takes as stride_ex = 1, stride_var = N.
#
# Indices: `example_ids` and categories are 0-based on the device side, as in the reference
# (src/nodes/fixable_categorical_dist.jl:43-44); the functions below take and return Julia's 1-based
# ranges where the reference does.
module PCMI355

include("LibPCMI355.jl")
using .LibPCMI355
using Random

export DeviceArray, to_device, to_host, Circuit, hclt, hclt_from_clt, compile_circuit, num_parameters,
       loglikelihoods, loglikelihood, probs_flows_circuit, mini_batch_em_with_reg, mini_batch_em_beta, mini_batch_em_for_multihead_pc,
       vectorize_parameters, update_parameters, kld, kld_backward, gumbel_sample, gumbel_sample_backward,
       per_sample_normalized_flows, normalize_params, pairwise_MI, learn_chow_liu_tree

# ---------------------------------------------------------------------------------------------- errors

struct PcmError <: Exception
    code::Cint
    msg::String
end
Base.showerror(io::IO, e::PcmError) = print(io, "libpcmi355 (", e.code, "): ", e.msg)

"Every entry point returns a status; anything but 0 is thrown with the library's message."
function check(rc::Integer)
    rc == 0 && return nothing
    throw(PcmError(Cint(rc), unsafe_string(LibPCMI355.pcm_last_error())))
end

# ---------------------------------------------------------------------------------------------- device memory

const libhip = get(ENV, "LIBAMDHIP64", "libamdhip64.so")
const hipMemcpyHostToDevice = Cint(1)
const hipMemcpyDeviceToHost = Cint(2)

function hipcheck(rc::Integer, what)
    rc == 0 || error("HIP call $what failed with status $rc")
    nothing
end

"A dense column-major array in device memory.  Freed by its finalizer."
mutable struct DeviceArray{T,N}
    ptr::Ptr{T}
    dims::NTuple{N,Int}
    function DeviceArray{T}(dims::Vararg{Integer,N}) where {T,N}
        p = Ref{Ptr{Cvoid}}(C_NULL)
        bytes = max(prod(dims) * sizeof(T), 16)
        hipcheck(ccall((:hipMalloc, libhip), Cint, (Ptr{Ptr{Cvoid}}, Csize_t), p, bytes), "hipMalloc")
        a = new{T,N}(Ptr{T}(p[]), map(Int, dims))
        finalizer(x -> ccall((:hipFree, libhip), Cint, (Ptr{Cvoid},), x.ptr), a)
        a
    end
end
Base.size(a::DeviceArray) = a.dims
Base.size(a::DeviceArray, i::Integer) = a.dims[i]
Base.length(a::DeviceArray) = prod(a.dims)
Base.eltype(::DeviceArray{T}) where {T} = T

"Device address of `x`; define a method for other device array types (e.g. `AMDGPU.ROCArray`)."
device_pointer(a::DeviceArray) = a.ptr
device_pointer(::Nothing) = C_NULL
"Address of the element at linear offset `off` (0-based)."
device_pointer(a, off::Integer) = device_pointer(a) + off * sizeof(eltype(a))

function to_device(h::Array{T,N}) where {T,N}
    d = DeviceArray{T}(size(h)...)
    hipcheck(ccall((:hipMemcpy, libhip), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t, Cint),
                   d.ptr, h, sizeof(h), hipMemcpyHostToDevice), "hipMemcpy")
    d
end
function to_host(d::DeviceArray{T,N}) where {T,N}
    h = Array{T,N}(undef, d.dims)
    hipcheck(ccall((:hipMemcpy, libhip), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t, Cint),
                   h, d.ptr, sizeof(h), hipMemcpyDeviceToHost), "hipMemcpy")
    h
end
device_sync() = hipcheck(ccall((:hipDeviceSynchronize, libhip), Cint, ()), "hipDeviceSynchronize")

# ---------------------------------------------------------------------------------------------- circuits

"A compiled circuit on the device: what `CuMetaBitsProbCircuit(pc)` / `CuMultiHeadBitsProbCircuit(pcs)` give the
reference (src/bits_circuit.jl:5-113, src-jl/multi_head_pc/bit_circuit.jl:4-56).  The library owns the memory."
mutable struct Circuit
    h::Ptr{Cvoid}
    num_vars::Int
    num_cats::Int
    num_heads::Int
    function Circuit(h, num_vars, num_cats, num_heads)
        c = new(h, num_vars, num_cats, num_heads)
        finalizer(x -> LibPCMI355.pcm_free(x.h), c)
        c
    end
end

"`hclt_from_clt` + compilation (src/structures/hclts.jl:100-145, src/bits_circuit.jl:39): `clt_parent[v]` is the
0-based parent of variable v in the Chow-Liu tree, -1 at the root.  `num_heads > 0`: the multi-head form."
function hclt_from_clt(clt_parent::Vector{Int32}, num_cats::Integer, num_hidden_cats::Integer; num_heads::Integer = 0)
    out = Ref{Ptr{Cvoid}}(C_NULL)
    if num_heads > 0
        check(LibPCMI355.pcm_hclt_create_multihead(clt_parent, length(clt_parent), num_hidden_cats, num_cats, num_heads, out))
    else
        check(LibPCMI355.pcm_hclt_create(clt_parent, length(clt_parent), num_hidden_cats, num_cats, out))
    end
    Circuit(out[], length(clt_parent), num_cats, num_heads)
end

"`pairwise_MI(data, num_cats; pseudocount)` (src/utils/information.jl:3-158) on the device; `data` is [N, V]."
function pairwise_MI(data, num_cats::Integer; pseudocount = 0.1)
    n, v = size(data)
    mi = DeviceArray{Float32}(v, v)
    check(LibPCMI355.pcm_pairwise_mi(device_pointer(data), 1, n, n, v, num_cats, pseudocount, device_pointer(mi), C_NULL))
    device_sync()
    mi
end

"`learn_chow_liu_tree` + `clt_edges2graphs` (src/structures/hclts.jl:17-18): parent array of the maximum spanning tree."
function learn_chow_liu_tree(mi::Matrix{Float32})
    v = size(mi, 1)
    parent = Vector{Int32}(undef, v)
    check(LibPCMI355.pcm_chow_liu_tree(mi, v, parent))
    parent
end

"`hclt(data, num_hidden_cats; num_cats, pseudocount)` (src/structures/hclts.jl:7-24)."
function hclt(data, num_hidden_cats::Integer; num_cats::Integer, pseudocount = 0.1, num_heads::Integer = 0)
    parent = learn_chow_liu_tree(to_host(pairwise_MI(data, num_cats; pseudocount = pseudocount)))
    hclt_from_clt(parent, num_cats, num_hidden_cats; num_heads = num_heads)
end

"Any circuit, as flat arrays in children-before-parents order (what walking a `ProbCircuit` DAG gives:
src/bits_circuit.jl:39-113; multi-head: the heads last, src-jl/multi_head_pc/bit_circuit.jl:14-56).
node_type: 0 input, 1 product, 2 sum; child_ptr / child_idx CSR (0-based); one log-parameter per sum edge;
input_var (0-based) and num_cats log-probabilities per input node."
function compile_circuit(node_type::Vector{UInt8}, child_ptr::Vector{Int32}, child_idx::Vector{Int32},
                         sum_logp::Vector{Float32}, input_var::Vector{Int32}, input_logp::Vector{Float32},
                         num_vars::Integer, num_cats::Integer; num_heads::Integer = 0)
    out = Ref{Ptr{Cvoid}}(C_NULL)
    check(LibPCMI355.pcm_circuit_create(length(node_type), node_type, child_ptr, child_idx, sum_logp, input_var,
                                        input_logp, num_vars, num_cats, num_heads, out))
    Circuit(out[], num_vars, num_cats, num_heads)
end

"`num_parameters(bpc)` (src/bits_circuit.jl:119-131)."
num_parameters(c::Circuit) = Int(LibPCMI355.pcm_size(c.h, 0))

"`vectorize_parameters(bpc)` (src/misc.jl:5-40): sum edges in up order, then the input nodes' tables."
function vectorize_parameters(c::Circuit)
    p = Vector{Float32}(undef, num_parameters(c))
    check(LibPCMI355.pcm_vectorize_parameters(c.h, p, length(p)))
    p
end

"`update_parameters(bpc, params)` (src/misc.jl:73-102)."
function update_parameters(c::Circuit, params::Vector{Float32})
    check(LibPCMI355.pcm_update_parameters(c.h, params, length(params)))
    nothing
end

# ---------------------------------------------------------------------------------------------- likelihoods

"`loglikelihoods(bpc, data; batch_size)` (src/regularization/reg_likelihood.jl:139-162): a device vector [N];
for a multi-head circuit without `head_mask` [N, H], with it [N] (src-jl/multi_head_pc/likelihood.jl:37-71).
`data` is a [N, V] UInt8 device matrix, `head_mask` a [N, H] Float32 device matrix."
function loglikelihoods(c::Circuit, data; batch_size::Integer, head_mask = nothing)
    n = size(data, 1)
    if c.num_heads > 0 && head_mask === nothing
        lls = DeviceArray{Float32}(n, c.num_heads)
        # the library writes [heads][batch] per call: with one call per batch the columns of a batch are n apart
        # only when the batch is the whole set, so batches go through a staging buffer
        stage = DeviceArray{Float32}(batch_size, c.num_heads)
        for s in 0:batch_size:n-1
            b = min(batch_size, n - s)
            check(LibPCMI355.pcm_loglikelihoods(c.h, device_pointer(data, s), 1, n, C_NULL, b, device_pointer(stage)))
            for h in 0:c.num_heads-1
                hipcheck(ccall((:hipMemcpy, libhip), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t, Cint),
                               device_pointer(lls, h * n + s), device_pointer(stage, h * b), b * sizeof(Float32), Cint(3)),
                         "hipMemcpy")
            end
        end
        return lls
    end
    if head_mask !== nothing   # the mixture of the heads, from the per-head values (src-jl/multi_head_pc/likelihood.jl:3-12)
        per_head = to_host(loglikelihoods(c, data; batch_size = batch_size))        # [N, H]
        hm = to_host(head_mask)
        mix = Vector{Float32}(undef, n)
        for e in 1:n
            t = per_head[e, :] .+ log.(hm[e, :])
            m = maximum(t)
            mix[e] = (isfinite(m) ? m + log(sum(exp.(t .- m))) : m) - log(sum(hm[e, :]))
        end
        return to_device(mix)
    end
    lls = DeviceArray{Float32}(n)
    for s in 0:batch_size:n-1
        b = min(batch_size, n - s)
        check(LibPCMI355.pcm_loglikelihoods(c.h, device_pointer(data, s), 1, n, C_NULL, b, device_pointer(lls, s)))
    end
    lls
end

"`loglikelihood(bpc, data; batch_size)`: the mean."
loglikelihood(c::Circuit, data; batch_size::Integer) = sum(to_host(loglikelihoods(c, data; batch_size = batch_size))) / size(data, 1)

# ---------------------------------------------------------------------------------------------- flows and EM

"`probs_flows_circuit(flows, edge_flows, ..., mbpc, data, example_ids; ...)` (src/queries/flow.jl:228-234) for one
batch: forward, backward, leaf flows.  The scratch arrays of the reference's signature are the library's own;
`example_ids` is a 0-based Int32 device vector (or nothing = the first `batch` rows), `rate` scales what the
accumulators held before (0 clears them, src/regularization/reg_em.jl:276-284).  Returns the batch's log-likelihoods."
function probs_flows_circuit(c::Circuit, data, example_ids; batch::Integer = length(example_ids), rate = 0f0,
                             head_mask = nothing, lls = DeviceArray{Float32}(batch))
    check(LibPCMI355.pcm_flows(c.h, device_pointer(data), 1, size(data, 1), device_pointer(example_ids), batch, rate,
                               device_pointer(head_mask), device_pointer(lls)))
    lls
end

"`mini_batch_em_with_reg(bpc, data, num_epochs; batch_size, pseudocount, soft_reg, soft_reg_width, ent_reg,
param_inertia, param_inertia_end, flow_memory, shuffle, verbose)` (src/regularization/reg_em.jl:208-336): the mean
log-likelihood of every epoch.  `soft_reg` > 0 is set on the handle for the length of the loop (`pcm_set_soft_reg`:
HCLT handles on the block kernels; `soft_flow_as_written` picks the leaf statistics of reg_flow.jl:12-17 as they
stand); `ent_reg` > 0 is refused (the reference has it commented out, reg_em.jl:294-296)."
function mini_batch_em_with_reg(c::Circuit, data, num_epochs::Integer; batch_size::Integer, pseudocount,
                                soft_reg = 0.0, soft_reg_width = 1, ent_reg = 0.0,
                                param_inertia, param_inertia_end = param_inertia, flow_memory = 0,
                                shuffle = :each_epoch, verbose = true, rng = Random.default_rng(),
                                soft_flow_as_written::Bool = true)
    @assert pseudocount >= 0
    ent_reg == 0 || throw(ArgumentError("ent_reg is not part of this path"))
    soft_reg == 0 || check(LibPCMI355.pcm_set_soft_reg(c.h, Float32(soft_reg), Int32(soft_reg_width), Int32(soft_flow_as_written)))
    n = size(data, 1)
    @assert batch_size <= n
    num_batches = n ÷ batch_size                                            # reg_em.jl:216
    ids_host = Vector{Int32}(undef, n)
    ids_host .= Int32.(0:n-1)
    shuffle == :once && shuffle!(rng, ids_host)                             # reg_em.jl:245-249
    ids = to_device(ids_host)
    lls = DeviceArray{Float32}(batch_size)
    log_likelihoods = Float32[]
    delta = (param_inertia_end - param_inertia) / num_epochs                # reg_em.jl:258
    inertia = Float32(param_inertia)
    for epoch in 1:num_epochs
        if shuffle == :each_epoch                                           # reg_em.jl:251-254
            shuffle!(rng, ids_host)
            ids = to_device(ids_host)
        end
        total = 0.0
        for batch_id in 0:num_batches-1
            rate = flow_memory > 0 ? max(0f0, 1f0 - Float32((batch_size + pseudocount) / flow_memory)) : 0f0   # reg_em.jl:281
            check(LibPCMI355.pcm_em_step(c.h, device_pointer(data), 1, n, device_pointer(ids, batch_id * batch_size),
                                         batch_size, rate, Float32(pseudocount), inertia, device_pointer(lls)))
            total += sum(to_host(lls))
        end
        push!(log_likelihoods, Float32(total / (num_batches * batch_size)))
        verbose && println("epoch ", epoch, ": train LL ", log_likelihoods[end])
        inertia += Float32(delta)                                           # reg_em.jl:307
    end
    soft_reg == 0 || check(LibPCMI355.pcm_set_soft_reg(c.h, 0f0, Int32(1), Int32(0)))
    log_likelihoods
end

"`mini_batch_em_beta(bpc, data, num_epochs; batch_size, pseudocount, soft_reg, soft_reg_width, param_inertia,
param_inertia_end, flow_memory, flow_memory_end, shuffle, update_interval, fscale, verbose)`
(VariationalJuice.jl/src-jl/learning/em.jl:289-409): statistics collect over `update_interval` batches -- cleared at the
start of an epoch, cleared or decayed by the flow memory at a batch with batch_id % update_interval == 1, every batch
adds its flows, the parameters move after a batch with batch_id % update_interval == 0 -- with schedules for the
inertia and the flow memory.  `fscale` other than 1: the flows of the tempered posterior (`pcm_set_flow_scale`); together
with `soft_reg` the library smooths through soft evidence and needs `soft_flow_as_written = false`."
function mini_batch_em_beta(c::Circuit, data, num_epochs::Integer; batch_size::Integer, pseudocount,
                            soft_reg = 0.0, soft_reg_width = 1, param_inertia, param_inertia_end = param_inertia,
                            flow_memory = 0, flow_memory_end = flow_memory, shuffle = :each_epoch,
                            update_interval::Integer = 1, fscale = 1.0, verbose = true, rng = Random.default_rng(),
                            soft_flow_as_written::Bool = true)
    @assert pseudocount >= 0
    @assert 0 <= param_inertia <= 1
    @assert param_inertia <= param_inertia_end <= 1
    @assert 0 <= flow_memory <= flow_memory_end                            # em.jl:299-303
    @assert update_interval >= 1
    n = size(data, 1)
    @assert batch_size <= n
    num_batches = n ÷ batch_size
    soft_reg == 0 || check(LibPCMI355.pcm_set_soft_reg(c.h, Float32(soft_reg), Int32(soft_reg_width), Int32(soft_flow_as_written)))
    fscale == 1 || check(LibPCMI355.pcm_set_flow_scale(c.h, Float32(fscale)))
    ids_host = Vector{Int32}(undef, n)
    ids_host .= Int32.(0:n-1)
    shuffle == :once && shuffle!(rng, ids_host)
    ids = to_device(ids_host)
    lls = DeviceArray{Float32}(batch_size)
    log_likelihoods = Float32[]
    delta = (param_inertia_end - param_inertia) / num_epochs
    delta_memory = (flow_memory_end - flow_memory) / num_epochs
    inertia = Float32(param_inertia)
    memory = Float64(flow_memory)
    for epoch in 1:num_epochs
        if shuffle == :each_epoch
            shuffle!(rng, ids_host)
            ids = to_device(ids_host)
        end
        total = 0.0
        cleared = true                                                      # em.jl:344-345
        for batch_id in 1:num_batches
            if shuffle == :each_batch
                shuffle!(rng, ids_host)
                ids = to_device(ids_host)
            end
            rate = 1f0
            if batch_id % update_interval == 1                              # em.jl:354-363
                rate = memory == 0 ? 0f0 : max(0f0, 1f0 - Float32((batch_size + pseudocount) / memory))
            end
            if cleared
                rate = 0f0
                cleared = false
            end
            check(LibPCMI355.pcm_flows(c.h, device_pointer(data), 1, n, device_pointer(ids, (batch_id - 1) * batch_size),
                                       batch_size, rate, device_pointer(nothing), device_pointer(lls)))
            total += sum(to_host(lls))
            if batch_id % update_interval == 0                              # em.jl:373-379
                check(LibPCMI355.pcm_em_update(c.h, Float32(pseudocount), inertia))
            end
        end
        push!(log_likelihoods, Float32(total / (num_batches * batch_size)))
        verbose && println("epoch ", epoch, ": train LL ", log_likelihoods[end])
        inertia += Float32(delta)
        memory += delta_memory
    end
    soft_reg == 0 || check(LibPCMI355.pcm_set_soft_reg(c.h, 0f0, Int32(1), Int32(0)))
    fscale == 1 || check(LibPCMI355.pcm_set_flow_scale(c.h, 1f0))
    log_likelihoods
end

"`mini_batch_em_for_multihead_pc(mhbpc, data, head_mask, num_epochs; ...)` (src-jl/multi_head_pc/em.jl:1-99)."
function mini_batch_em_for_multihead_pc(c::Circuit, data, head_mask, num_epochs::Integer; batch_size::Integer, pseudocount,
                                        param_inertia, param_inertia_end = param_inertia, flow_memory = 0,
                                        shuffle = :each_epoch, verbose = true, rng = Random.default_rng())
    @assert c.num_heads > 0
    n = size(data, 1)
    num_batches = n ÷ batch_size
    order = collect(0:n-1)
    lls = DeviceArray{Float32}(batch_size)
    log_likelihoods = Float32[]
    delta = (param_inertia_end - param_inertia) / num_epochs
    inertia = Float32(param_inertia)
    mask_host = to_host(head_mask)                                         # [N, H]
    shuffle == :once && shuffle!(rng, order)
    for epoch in 1:num_epochs
        shuffle == :each_epoch && shuffle!(rng, order)
        total = 0.0
        for batch_id in 0:num_batches-1
            rows = order[batch_id*batch_size+1:(batch_id+1)*batch_size]
            ids = to_device(Int32.(rows))
            mask_b = to_device(Matrix{Float32}(mask_host[rows.+1, :]))      # [batch, H] column-major = [heads][batch]
            rate = flow_memory > 0 ? max(0f0, 1f0 - Float32((batch_size + pseudocount) / flow_memory)) : 0f0
            # (pcm_em_step has no mask argument: masked flows and the update are two calls)
            check(LibPCMI355.pcm_flows(c.h, device_pointer(data), 1, n, device_pointer(ids), batch_size, rate,
                                       device_pointer(mask_b), device_pointer(lls)))
            check(LibPCMI355.pcm_em_update(c.h, Float32(pseudocount), inertia))
            total += sum(to_host(lls))
        end
        push!(log_likelihoods, Float32(total / (num_batches * batch_size)))
        verbose && println("epoch ", epoch, ": train LL ", log_likelihoods[end])
        inertia += Float32(delta)
    end
    log_likelihoods
end

# ---------------------------------------------------------------------------------------------- KL, sampling

"`kld(mbpc, params1, params2; norm_params)` (src/queries/kld.jl:164-206): `params` are [rows, n] Float32 device
matrices in `vectorize_parameters` order; returns klds[:, end] as a device vector [rows]."
function kld(c::Circuit, params1, params2; norm_params::Bool = false)
    r = size(params1, 1)
    klds = DeviceArray{Float32}(r)
    check(LibPCMI355.pcm_kld_rows(c.h, device_pointer(params1), device_pointer(params2), 1, r, r, norm_params, device_pointer(klds)))
    klds
end

"`kld_backward(mbpc, params1, params2; norm_params, grad_wrt_logparams = true)` (src/queries/kld.jl:593-649)."
function kld_backward(c::Circuit, params1, params2; norm_params::Bool = false)
    r, n = size(params1)
    g1 = DeviceArray{Float32}(r, n)
    g2 = DeviceArray{Float32}(r, n)
    check(LibPCMI355.pcm_kld_backward_rows(c.h, device_pointer(params1), device_pointer(params2), 1, r, r, norm_params,
                                           device_pointer(g1), device_pointer(g2), C_NULL))
    g1, g2
end

"`gumbel_sample(mbpc, params, num_vars, par_buffer_size; temperature, no_gumbel, norm_params)`
(src/queries/sample.jl:338-383) with the noise supplied (`noise` = nothing: no_gumbel): the soft assignment
[num_cats, num_vars, rows] in memory, i.e. [rows][vars][cats]."
function gumbel_sample(c::Circuit, params; temperature, noise = nothing, norm_params::Bool = false)
    r = size(params, 1)
    out = DeviceArray{Float32}(c.num_cats, c.num_vars, r)
    check(LibPCMI355.pcm_gumbel_sample_rows(c.h, device_pointer(params), 1, r, r, device_pointer(noise), temperature,
                                            norm_params, device_pointer(out)))
    out
end

"`gumbel_sample_backward(mbpc, params, input_aggr_params, input_aggr_grads, temperature; norm_params,
grad_wrt_logparams)` (src/queries/sample.jl:620-692)."
function gumbel_sample_backward(c::Circuit, params, out_grads; temperature, noise = nothing, norm_params::Bool = false,
                                grad_wrt_logparams::Bool = true)
    r, n = size(params)
    g = DeviceArray{Float32}(r, n)
    check(LibPCMI355.pcm_gumbel_sample_backward_rows(c.h, device_pointer(params), 1, r, r, device_pointer(noise), temperature,
                                                     norm_params, grad_wrt_logparams, device_pointer(out_grads), device_pointer(g)))
    g
end

# ---------------------------------------------------------------------------------------------- per-example flows

"`per_sample_normalized_flows(mbpc, data; batch_size)` (src/queries/flow.jl:417-464): [N, num_parameters]."
function per_sample_normalized_flows(c::Circuit, data; batch_size::Integer, as_written::Bool = true)
    n = size(data, 1)
    np = num_parameters(c)
    out = DeviceArray{Float32}(n, np)
    for s in 0:batch_size:n-1
        b = min(batch_size, n - s)
        check(LibPCMI355.pcm_normalized_flows(c.h, device_pointer(data, s), 1, n, C_NULL, b, as_written,
                                              device_pointer(out, s), 1, n))
    end
    out
end

"`normalize_params(mbpc, params; undo)` (src/misc.jl:448) on a [rows, n] device matrix, in place."
function normalize_params(c::Circuit, params; undo::Bool = false)
    r = size(params, 1)
    check(LibPCMI355.pcm_normalize_params_rows(c.h, device_pointer(params), 1, r, r, undo))
    params
end

end # module
