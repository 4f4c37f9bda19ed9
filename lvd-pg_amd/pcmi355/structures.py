"""Structure learning: the step before `hclt_from_clt`, named after the reference functions."""
import numpy as np
import torch

from ._lib import lib, check, np_ptr
from .circuits import hclt_from_clt


def pairwise_MI(data, num_cats=None, pseudocount=0.1):
    """`pairwise_MI_chunked(data; num_cats, pseudocount)` (src/utils/information.jl:97-141):
    mutual information of every pair of variables of a uint8 device tensor [N, V]; returns a
    float32 device tensor [V, V] (symmetric, diagonal included).  No chunking is needed: a
    pair's table never leaves the workgroup that counts it."""
    if not (isinstance(data, torch.Tensor) and data.is_cuda and data.dtype == torch.uint8 and data.dim() == 2):
        raise ValueError("data must be a 2-D uint8 tensor on the GPU (examples x variables)")
    n, v = data.shape
    if num_cats is None:
        num_cats = int(data.max().item()) + 1
    mi = torch.empty((v, v), dtype=torch.float32, device=data.device)
    check(lib.pcm_pairwise_mi(data.data_ptr(), data.stride(0), data.stride(1), n, v, int(num_cats), float(pseudocount),
                              mi.data_ptr(), torch.cuda.current_stream(data.device).cuda_stream))
    return mi


def chow_liu_tree(mi):
    """Maximum spanning tree of a mutual-information matrix, directed away from the centre of
    the tree (what `learn_chow_liu_tree` followed by `clt_edges2graphs(...; shape = :directed)`
    gives src/structures/hclts.jl:17-18), as the parent array `hclt_from_clt` takes."""
    m = np.ascontiguousarray(mi.detach().cpu().numpy() if isinstance(mi, torch.Tensor) else mi, dtype=np.float32)
    if m.ndim != 2 or m.shape[0] != m.shape[1]:
        raise ValueError("mi must be a square matrix")
    parent = np.empty(m.shape[0], np.int32)
    check(lib.pcm_chow_liu_tree(np_ptr(m), m.shape[0], np_ptr(parent)))
    return parent


def learn_chow_liu_tree(data, num_cats=None, pseudocount=0.1):
    """`learn_chow_liu_tree(data; pseudocount)` as src/structures/hclts.jl:17 calls it, returning
    the rooted tree as a parent array."""
    return chow_liu_tree(pairwise_MI(data, num_cats, pseudocount))


def hclt(data, num_hidden_cats, num_cats=None, pseudocount=0.1):
    """`hclt(data, num_hidden_cats; num_cats, pseudocount)` (src/structures/hclts.jl:7-24) with
    one variable per group: Chow-Liu tree of the data, then the hidden Chow-Liu tree circuit."""
    if num_cats is None:
        num_cats = int(data.max().item()) + 1
    return hclt_from_clt(learn_chow_liu_tree(data, num_cats, pseudocount), int(num_cats), int(num_hidden_cats))
