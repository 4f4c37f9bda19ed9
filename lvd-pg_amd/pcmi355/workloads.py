"""Synthetic workloads of the benchmark configurations: seeded Gaussian-random-field
images, a Chow-Liu tree over them, and seeded parameter draws.  Host-side numpy; this is
benchmark input preparation, not part of the timed path.

Two trees: `make_config(name, tree="chow_liu")` learns it as the reference does
(`learn_chow_liu_tree(data; pseudocount = 0.1)` + `clt_edges2graphs`, src/structures/hclts.jl:17-18)
with the library's own pairwise mutual information and spanning tree, on a training set of
TRAIN_EXAMPLES images of which the batch is the head; it needs the GPU.  `tree="gaussian"` (the
default, host only) takes the mutual information from the Gaussian closed form
-0.5*log(1 - rho^2) of the pixel correlations of the batch; the maximum spanning tree is exact and
the root is the tree's centre.
"""
import numpy as np


def grf_images(n, height, width, channels, lengthscale, channel_corr=0.8, seed=0):
    """uint8 [n, channels*height*width]; variable index = c*H*W + h*W + w (the layout of
    `group_vars_by_grid`, src/structures/hclts.jl:189-224).  White noise is filtered in the
    Fourier domain with a squared-exponential kernel; channel i is
    sqrt(corr)*g0 + sqrt(1-corr)*g_i; the whole dataset is min-max quantised to 0..255."""
    rng = np.random.default_rng(seed)
    fy = np.fft.fftfreq(height)[:, None]
    fx = np.fft.rfftfreq(width)[None, :]
    filt = np.exp(-2.0 * (np.pi * lengthscale) ** 2 * (fx ** 2 + fy ** 2))

    def field(count):
        w = rng.standard_normal((count, height, width)).astype(np.float32)
        f = np.fft.irfft2(np.fft.rfft2(w) * filt, s=(height, width)).astype(np.float32)
        return f / f.std()

    base = field(n)
    out = np.empty((n, channels, height, width), np.float32)
    if channels == 1:
        out[:, 0] = base
    else:
        for c in range(channels):
            out[:, c] = np.sqrt(channel_corr) * base + np.sqrt(1.0 - channel_corr) * field(n)
    lo, hi = out.min(), out.max()
    q = np.clip(np.floor((out - lo) / (hi - lo) * 256.0), 0, 255).astype(np.uint8)
    return q.reshape(n, channels * height * width)


def chow_liu_parent(data):
    """Parent array (root = -1) of the maximum spanning tree of Gaussian mutual
    information, rooted at the tree centre.  Ties are broken by variable index."""
    from scipy.sparse.csgraph import minimum_spanning_tree, breadth_first_order
    x = data.astype(np.float32)
    V = x.shape[1]
    x -= x.mean(axis=0, keepdims=True)
    sd = x.std(axis=0, keepdims=True)
    x /= np.where(sd > 0, sd, 1)
    rho = (x.T @ x) / x.shape[0]
    np.clip(rho, -0.999999, 0.999999, out=rho)
    mi = -0.5 * np.log1p(-rho.astype(np.float64) ** 2)
    w = (mi.max() + 1e-6) - mi          # positive weights, small = strong dependence
    np.fill_diagonal(w, 0)
    mst = minimum_spanning_tree(w)
    adj = mst + mst.T

    def farthest(src):
        order, pred = breadth_first_order(adj, src, directed=False, return_predecessors=True)
        depth = np.zeros(V, np.int64)
        for v in order[1:]:
            depth[v] = depth[pred[v]] + 1
        return int(np.argmax(depth)), pred, depth

    a, _, _ = farthest(0)
    b, pred, depth = farthest(a)
    path = [b]
    while path[-1] != a:
        path.append(int(pred[path[-1]]))
    root = path[len(path) // 2]
    order, pred = breadth_first_order(adj, root, directed=False, return_predecessors=True)
    parent = np.where(pred < 0, -1, pred).astype(np.int32)
    parent[root] = -1
    return parent


def tree_stats(parent):
    V = len(parent)
    nchild = np.zeros(V, np.int64)
    for v in range(V):
        if parent[v] >= 0:
            nchild[parent[v]] += 1
    depth = np.zeros(V, np.int64)
    order = np.argsort(parent, kind="stable")
    # depth by repeated relaxation along parent pointers (tree is shallow relative to V)
    changed = True
    while changed:
        nd = np.where(parent >= 0, depth[np.maximum(parent, 0)] + 1, 0)
        changed = bool((nd != depth).any())
        depth = nd
    return dict(n_inner=int((nchild > 0).sum()), n_leaf=int((nchild == 0).sum()), depth=int(depth.max()),
                max_children=int(nchild.max()))


def init_params(parent, K, C, seed, kind="perturb"):
    """Seeded parameters in block form (theta [V,K,K], leaf [V,K,C], log space).
    kind='perturb': uniform(0.6, 1.4) normalised == init_parameters(perturbation = 0.4)
    (src/nodes/fixable_categorical_dist.jl:31-37); kind='dirichlet': Dirichlet(1)."""
    rng = np.random.default_rng(seed)
    V = len(parent)

    def draw(shape):
        if kind == "dirichlet":
            x = rng.exponential(size=shape).astype(np.float32)
        else:
            x = rng.uniform(0.6, 1.4, size=shape).astype(np.float32)
        x = np.maximum(x, 1e-30)
        return np.log(x / x.sum(axis=-1, keepdims=True)).astype(np.float32)

    return draw((V, K, K)), draw((V, K, C))


CONFIGS = {
    # name: (height, width, channels, K, C, batch, lengthscale, seed)
    "c1_hclt64_k16": (8, 8, 1, 16, 256, 1024, 2.0, 1001),
    "c3_hclt3072_k32": (32, 32, 3, 32, 256, 4096, 3.0, 1003),
}


TRAIN_EXAMPLES = 32768      # images the Chow-Liu tree of tree="chow_liu" is learned from


def make_config(name, tree="gaussian"):
    h, w, ch, K, C, B, ls, seed = CONFIGS[name]
    if tree == "chow_liu":
        import torch
        from .structures import learn_chow_liu_tree
        train = grf_images(TRAIN_EXAMPLES, h, w, ch, ls, 0.8, seed)
        parent = learn_chow_liu_tree(torch.from_numpy(train).cuda(), C, 0.1)
        data = np.ascontiguousarray(train[:B])
        del train
    elif tree == "gaussian":
        data = grf_images(B, h, w, ch, ls, 0.8, seed)
        parent = chow_liu_parent(data)
    else:
        raise ValueError("tree: 'gaussian' or 'chow_liu'")
    theta, leaf = init_params(parent, K, C, seed + 100)
    return dict(name=name, data=data, parent=parent, theta=theta, leaf=leaf, K=K, C=C, B=B, V=h * w * ch)


def c2_config():
    """The K = 128 configuration: 48 variables (one 4x4x3 patch, 256 categories), Dirichlet(1) parameters, batch
    4096 of smoothed-random-field patches with channel correlation 0.8."""
    V, K, C, B = 48, 128, 256, 4096
    data = grf_images(B, 4, 4, 3, 2.0, 0.8, seed=1002)
    parent = chow_liu_parent(data)
    theta, leaf = init_params(parent, K, C, 1102, kind="dirichlet")
    return dict(name="c2_hclt48_k128", data=data, parent=parent, theta=theta, leaf=leaf, K=K, C=C, B=B, V=V)


def c4_config(batch=1024):
    """The patch-clustered configuration: 64 x 64 x 3 images cut into 64 patches of 8 x 8 x 3; one 192-variable
    K = 32 circuit with 128 cluster heads per patch, all of them as one forest over the 12288 pixels, seeded
    uniform cluster ids per (image, patch), and the K = 64 top-level tree over the 64 cluster ids.
    Returns the per-patch pieces (`pvars`, `parents`, `params`) and the forest's arrays: `fparent` (64 roots),
    `theta`, `leaf` indexed by pixel, `mask` [trees][heads][batch] one-hot in the forest's tree order (trees are
    numbered by their root's variable), `tree_patch[t]` = the patch tree t covers."""
    V, K, C, H, NP = 192, 32, 256, 128, 64
    rng = np.random.default_rng(0)
    img = grf_images(batch, 64, 64, 3, 3.0, 0.8, seed=1004).reshape(batch, 3, 64, 64)
    pixel = np.arange(3 * 64 * 64).reshape(3, 64, 64)
    pvars = [pixel[:, 8 * (p // 8):8 * (p // 8) + 8, 8 * (p % 8):8 * (p % 8) + 8].reshape(V) for p in range(NP)]
    flat = np.ascontiguousarray(img.reshape(batch, -1))
    cluster = rng.integers(0, H, size=(batch, NP)).astype(np.uint8)
    parents = [chow_liu_parent(np.ascontiguousarray(flat[:, pv])) for pv in pvars]
    params = [init_params(parents[p], K, C, 2000 + p, kind="dirichlet") for p in range(NP)]
    nv = flat.shape[1]
    fparent = np.empty(nv, np.int32)
    theta = np.zeros((nv, K, K), np.float32)
    leaf = np.zeros((nv, K, C), np.float32)
    for pv, par, (th, lf) in zip(pvars, parents, params):
        fparent[pv] = np.where(par < 0, -1, pv[np.maximum(par, 0)])
        theta[pv], leaf[pv] = th, lf
    roots = [int(pv[np.flatnonzero(par < 0)[0]]) for pv, par in zip(pvars, parents)]
    tree_patch = np.argsort(roots)
    mask = np.zeros((NP, H, batch), np.float32)
    for t, p in enumerate(tree_patch):
        mask[t, cluster[:, p], np.arange(batch)] = 1.0
    tparent = chow_liu_parent(cluster)
    return dict(V=V, K=K, C=C, H=H, B=batch, patches=NP, data=flat, cluster=cluster, pvars=pvars, parents=parents,
                params=params, fparent=fparent, theta=theta, leaf=leaf, mask=mask, tree_patch=tree_patch,
                top_parent=tparent, top_params=init_params(tparent, 64, H, 2100, kind="dirichlet"))
