"""Host-side mirror of the reference's probabilistic-circuit API over libpcmi355.so.

The reference's host language (Julia) is not available where this package is built, so
the host side is Python; names, argument meaning and error behaviour follow the Julia
functions cited in each docstring (paths relative to VariationalJuice.jl/).  Device
memory and streams come from torch; everything numeric happens in the HIP library.
"""
from .circuits import (BitsCircuit, HcltCircuit, HcltForest, hclt_from_clt, multihead_hclt_from_clt,  # noqa: F401
                       hclt_forest_from_clts, compile_circuit,
                       compile_multihead, CuBitsProbCircuit, CuMultiHeadBitsProbCircuit, node_maps, write_back_parameters)
from .queries import (loglikelihoods, loglikelihood, loglikelihoods_probcat, loglikelihood_probcat, weighted_ll,
                      probs_flows_circuit, mini_batch_em_with_reg, mini_batch_em, mini_batch_em_beta,  # noqa: F401
                      vectorize_parameters, update_parameters, kld, kld_backward, sample, adam_step,
                      mini_batch_em_for_multihead_pc, multihead_loglikelihoods, gumbel_sample, gumbel_sample_rows, gumbel_sample_backward_rows,
                      patch_level_evidence, flow_gradients, adam, soft_reg_evidence, forest_loglikelihoods, forest_flows,
                      mini_batch_em_for_forest, per_sample_normalized_flows, normalize_params, map_pc_parameters)
from .structures import (pairwise_MI, chow_liu_tree, learn_chow_liu_tree, hclt, hclt_for_colored_images, clt_edges2parent, hclt_pc,  # noqa: F401
                         customized_hclt, joined_hclt, joined_hclt_from_clts, group_vars_by_grid, group_vars_by_cgrid)
from .transformations import prune_pc, grow_heads_by_flows, aggregate_edge_flows, aggregate_node_flows  # noqa: F401
from .jpc_io import write_jpc, read_jpc, write_mhpc, read_mhpc  # noqa: F401
from . import nodes, prealloc  # noqa: F401
from ._lib import PcmError, LIB_PATH  # noqa: F401
