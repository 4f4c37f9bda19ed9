# Raw bindings of libpcmi355.so: one function per entry point of include/pcmi355.h, same name, same
# arguments.  Written by gen_bindings.py from the header; do not edit by hand.
#
# Pointers named d_* are device addresses (e.g. `Ptr{Float32}(UInt(pointer(x)))` of a ROCArray), the others
# are host arrays or `Ref`s; a null pointer is `C_NULL`.  Status codes are those of `enum pcm_status`;
# `pcm_last_error()` has the message of the last failure on the calling thread.
module LibPCMI355

const libpcmi355 = get(ENV, "LIBPCMI355", joinpath(@__DIR__, "..", "libpcmi355.so"))

pcm_last_error() =
    ccall((:pcm_last_error, libpcmi355), Cstring, ())
pcm_version() =
    ccall((:pcm_version, libpcmi355), Cint, ())
pcm_hclt_create(clt_parent, num_vars, num_hidden_cats, num_cats, out) =
    ccall((:pcm_hclt_create, libpcmi355), Cint, (Ptr{Int32}, Int32, Int32, Int32, Ptr{Ptr{Cvoid}}), clt_parent, num_vars, num_hidden_cats, num_cats, out)
pcm_hclt_create_multihead(clt_parent, num_vars, num_hidden_cats, num_cats, num_heads, out) =
    ccall((:pcm_hclt_create_multihead, libpcmi355), Cint, (Ptr{Int32}, Int32, Int32, Int32, Int32, Ptr{Ptr{Cvoid}}), clt_parent, num_vars, num_hidden_cats, num_cats, num_heads, out)
pcm_hclt_create_forest(clt_parent, num_vars, num_hidden_cats, num_cats, num_heads, out) =
    ccall((:pcm_hclt_create_forest, libpcmi355), Cint, (Ptr{Int32}, Int32, Int32, Int32, Int32, Ptr{Ptr{Cvoid}}), clt_parent, num_vars, num_hidden_cats, num_cats, num_heads, out)
pcm_set_missing_category(c, on) =
    ccall((:pcm_set_missing_category, libpcmi355), Cint, (Ptr{Cvoid}, Int32), c, on)
pcm_set_soft_reg(c, soft_reg, soft_reg_width, as_written) =
    ccall((:pcm_set_soft_reg, libpcmi355), Cint, (Ptr{Cvoid}, Float32, Int32, Int32), c, soft_reg, soft_reg_width, as_written)
pcm_set_flow_scale(c, fscale) =
    ccall((:pcm_set_flow_scale, libpcmi355), Cint, (Ptr{Cvoid}, Float32), c, fscale)
pcm_hclt_set_heads(c, heads) =
    ccall((:pcm_hclt_set_heads, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Float32}), c, heads)
pcm_hclt_get_heads(c, heads) =
    ccall((:pcm_hclt_get_heads, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Float32}), c, heads)
pcm_circuit_create(num_nodes, node_type, child_ptr, child_idx, sum_logp, input_var, input_logp, num_vars, num_cats, num_heads, out) =
    ccall((:pcm_circuit_create, libpcmi355), Cint, (Int32, Ptr{UInt8}, Ptr{Int32}, Ptr{Int32}, Ptr{Float32}, Ptr{Int32}, Ptr{Float32}, Int32, Int32, Int32, Ptr{Ptr{Cvoid}}), num_nodes, node_type, child_ptr, child_idx, sum_logp, input_var, input_logp, num_vars, num_cats, num_heads, out)
pcm_free(c) =
    ccall((:pcm_free, libpcmi355), Cint, (Ptr{Cvoid},), c)
pcm_set_stream(c, hip_stream) =
    ccall((:pcm_set_stream, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Cvoid}), c, hip_stream)
pcm_size(c, what) =
    ccall((:pcm_size, libpcmi355), Int64, (Ptr{Cvoid}, Int32), c, what)
pcm_index_table(c, which, out, n) =
    ccall((:pcm_index_table, libpcmi355), Cint, (Ptr{Cvoid}, Int32, Ptr{Int64}, Int64), c, which, out, n)
pcm_vectorize_parameters(c, out, n) =
    ccall((:pcm_vectorize_parameters, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Float32}, Int64), c, out, n)
pcm_update_parameters(c, params, n) =
    ccall((:pcm_update_parameters, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Float32}, Int64), c, params, n)
pcm_hclt_set_params(c, theta, leaf) =
    ccall((:pcm_hclt_set_params, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Float32}, Ptr{Float32}), c, theta, leaf)
pcm_hclt_get_params(c, theta, leaf) =
    ccall((:pcm_hclt_get_params, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Float32}, Ptr{Float32}), c, theta, leaf)
pcm_hclt_get_flows(c, edge_aggr, leaf_flow) =
    ccall((:pcm_hclt_get_flows, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Float32}, Ptr{Float32}), c, edge_aggr, leaf_flow)
pcm_loglikelihoods(c, d_data, stride_ex, stride_var, d_example_ids, batch, d_ll_out) =
    ccall((:pcm_loglikelihoods, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{UInt8}, Int64, Int64, Ptr{Int32}, Int32, Ptr{Float32}), c, d_data, stride_ex, stride_var, d_example_ids, batch, d_ll_out)
pcm_flows(c, d_data, stride_ex, stride_var, d_example_ids, batch, rate, d_head_mask, d_ll_out) =
    ccall((:pcm_flows, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{UInt8}, Int64, Int64, Ptr{Int32}, Int32, Float32, Ptr{Float32}, Ptr{Float32}), c, d_data, stride_ex, stride_var, d_example_ids, batch, rate, d_head_mask, d_ll_out)
pcm_em_update(c, pseudocount, inertia) =
    ccall((:pcm_em_update, libpcmi355), Cint, (Ptr{Cvoid}, Float32, Float32), c, pseudocount, inertia)
pcm_em_step(c, d_data, stride_ex, stride_var, d_example_ids, batch, rate, pseudocount, inertia, d_ll_out) =
    ccall((:pcm_em_step, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{UInt8}, Int64, Int64, Ptr{Int32}, Int32, Float32, Float32, Float32, Ptr{Float32}), c, d_data, stride_ex, stride_var, d_example_ids, batch, rate, pseudocount, inertia, d_ll_out)
pcm_get_node_values(c, mars, flows, n) =
    ccall((:pcm_get_node_values, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Float32}, Ptr{Float32}, Int64), c, mars, flows, n)
pcm_node_flow_sums(c, out, n) =
    ccall((:pcm_node_flow_sums, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Float32}, Int64), c, out, n)
pcm_get_aggregates(c, edge_aggr, n_edges, leaf_flow, n_leaf) =
    ccall((:pcm_get_aggregates, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Float32}, Int64, Ptr{Float32}, Int64), c, edge_aggr, n_edges, leaf_flow, n_leaf)
pcm_kld(p, q, out) =
    ccall((:pcm_kld, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Float32}), p, q, out)
pcm_kld_backward(p, q, grad_p, grad_q, n) =
    ccall((:pcm_kld_backward, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Float32}, Ptr{Float32}, Int64), p, q, grad_p, grad_q, n)
pcm_kld_backward_dev(p, q, d_grad_p, d_grad_q, n) =
    ccall((:pcm_kld_backward_dev, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Float32}, Ptr{Float32}, Int64), p, q, d_grad_p, d_grad_q, n)
pcm_sample_noise_size(c) =
    ccall((:pcm_sample_noise_size, libpcmi355), Int64, (Ptr{Cvoid},), c)
pcm_sample(c, d_node_noise, d_leaf_noise, batch, d_out) =
    ccall((:pcm_sample, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Float32}, Ptr{Float32}, Int32, Ptr{UInt8}), c, d_node_noise, d_leaf_noise, batch, d_out)
pcm_sample_soft(c, d_node_noise, temperature, batch, d_out) =
    ccall((:pcm_sample_soft, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Float32}, Float32, Int32, Ptr{Float32}), c, d_node_noise, temperature, batch, d_out)
pcm_kld_rows(c, d_params1, d_params2, stride_row, stride_param, rows, norm_params, d_klds) =
    ccall((:pcm_kld_rows, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Float32}, Ptr{Float32}, Int64, Int64, Int32, Int32, Ptr{Float32}), c, d_params1, d_params2, stride_row, stride_param, rows, norm_params, d_klds)
pcm_kld_backward_rows(c, d_params1, d_params2, stride_row, stride_param, rows, norm_params, d_grads1, d_grads2, d_klds) =
    ccall((:pcm_kld_backward_rows, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Float32}, Ptr{Float32}, Int64, Int64, Int32, Int32, Ptr{Float32}, Ptr{Float32}, Ptr{Float32}), c, d_params1, d_params2, stride_row, stride_param, rows, norm_params, d_grads1, d_grads2, d_klds)
pcm_gumbel_sample_rows(c, d_params, stride_row, stride_param, rows, d_noise, temperature, norm_params, d_out) =
    ccall((:pcm_gumbel_sample_rows, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Float32}, Int64, Int64, Int32, Ptr{Float32}, Float32, Int32, Ptr{Float32}), c, d_params, stride_row, stride_param, rows, d_noise, temperature, norm_params, d_out)
pcm_gumbel_sample_backward_rows(c, d_params, stride_row, stride_param, rows, d_noise, temperature, norm_params, grad_wrt_logparams, d_out_grads, d_param_grads) =
    ccall((:pcm_gumbel_sample_backward_rows, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Float32}, Int64, Int64, Int32, Ptr{Float32}, Float32, Int32, Int32, Ptr{Float32}, Ptr{Float32}), c, d_params, stride_row, stride_param, rows, d_noise, temperature, norm_params, grad_wrt_logparams, d_out_grads, d_param_grads)
pcm_normalized_flows(c, d_data, stride_ex, stride_var, d_example_ids, batch, as_written, d_out, stride_row, stride_param) =
    ccall((:pcm_normalized_flows, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{UInt8}, Int64, Int64, Ptr{Int32}, Int32, Int32, Ptr{Float32}, Int64, Int64), c, d_data, stride_ex, stride_var, d_example_ids, batch, as_written, d_out, stride_row, stride_param)
pcm_normalize_params_rows(c, d_params, stride_row, stride_param, rows, undo) =
    ccall((:pcm_normalize_params_rows, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Float32}, Int64, Int64, Int32, Int32), c, d_params, stride_row, stride_param, rows, undo)
pcm_loglikelihoods_soft(c, d_evidence, stride_ex, stride_var, stride_cat, d_example_ids, batch, d_ll) =
    ccall((:pcm_loglikelihoods_soft, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Float32}, Int64, Int64, Int64, Ptr{Int32}, Int32, Ptr{Float32}), c, d_evidence, stride_ex, stride_var, stride_cat, d_example_ids, batch, d_ll)
pcm_flows_soft(c, d_evidence, stride_ex, stride_var, stride_cat, d_example_ids, batch, rate, d_head_mask, d_ll) =
    ccall((:pcm_flows_soft, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Float32}, Int64, Int64, Int64, Ptr{Int32}, Int32, Float32, Ptr{Float32}, Ptr{Float32}), c, d_evidence, stride_ex, stride_var, stride_cat, d_example_ids, batch, rate, d_head_mask, d_ll)
pcm_pairwise_mi(d_data, stride_ex, stride_var, num_examples, num_vars, num_cats, pseudocount, d_mi, stream) =
    ccall((:pcm_pairwise_mi, libpcmi355), Cint, (Ptr{UInt8}, Int64, Int64, Int64, Int32, Int32, Float32, Ptr{Float32}, Ptr{Cvoid}), d_data, stride_ex, stride_var, num_examples, num_vars, num_cats, pseudocount, d_mi, stream)
pcm_chow_liu_tree(mi, num_vars, clt_parent) =
    ccall((:pcm_chow_liu_tree, libpcmi355), Cint, (Ptr{Float32}, Int32, Ptr{Int32}), mi, num_vars, clt_parent)
pcm_pairwise_mi_static(d_data, stride_ex, stride_var, num_examples, num_vars, num_cats, pseudocount, d_mi, stream) =
    ccall((:pcm_pairwise_mi_static, libpcmi355), Cint, (Ptr{UInt8}, Int64, Int64, Int64, Int32, Int32, Float32, Ptr{Float32}, Ptr{Cvoid}), d_data, stride_ex, stride_var, num_examples, num_vars, num_cats, pseudocount, d_mi, stream)
pcm_adam_step(c, d_grad, d_params, d_m, d_v, lr, beta1, beta2, eps, t) =
    ccall((:pcm_adam_step, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Float32}, Ptr{Float32}, Ptr{Float32}, Ptr{Float32}, Float32, Float32, Float32, Float32, Int32), c, d_grad, d_params, d_m, d_v, lr, beta1, beta2, eps, t)
pcm_flow_gradients(c, batch_size, d_grad) =
    ccall((:pcm_flow_gradients, libpcmi355), Cint, (Ptr{Cvoid}, Int32, Ptr{Float32}), c, batch_size, d_grad)
pcm_adam_flow_step(c, batch_size, d_params, d_m, d_v, d_leaf_params, d_leaf_m, d_leaf_v, lr, beta1, beta2, eps, t) =
    ccall((:pcm_adam_flow_step, libpcmi355), Cint, (Ptr{Cvoid}, Int32, Ptr{Float32}, Ptr{Float32}, Ptr{Float32}, Ptr{Float32}, Ptr{Float32}, Ptr{Float32}, Float32, Float32, Float32, Float32, Int32), c, batch_size, d_params, d_m, d_v, d_leaf_params, d_leaf_m, d_leaf_v, lr, beta1, beta2, eps, t)
pcm_set_timing(c, on) =
    ccall((:pcm_set_timing, libpcmi355), Cint, (Ptr{Cvoid}, Int32), c, on)
pcm_get_timing(c, ms, n) =
    ccall((:pcm_get_timing, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Float32}, Int32), c, ms, n)
pcm_stream_probe(d_src, d_dst, lanes, reads, writes, grid, stream) =
    ccall((:pcm_stream_probe, libpcmi355), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Int64, Int32, Int32, Int32, Ptr{Cvoid}), d_src, d_dst, lanes, reads, writes, grid, stream)

end # module
