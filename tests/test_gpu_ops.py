"""The torch-facing operators and the Convolution module on the GPU, against the CPU oracle."""

import warnings

import numpy as np
import pytest
import torch

import e3j_amd
from e3j_amd import Convolution, ConvolutionParams, GraphOrdering, convolution, convolution_bwd
from e3j_amd.harmonics import Harmonics
from oracle import conv_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu


def dev(a, **kw):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda().requires_grad_(kw.get("grad", False))


def _problem(seed, N=12, E=70, X=5, Y=6, Z=7, S=4, K=16, nnz=60, sort_by="receiver", dtype=np.float32):
    rng = np.random.default_rng(seed)
    idx, val, mix = H.random_table(rng, nnz, X, Y, Z, S)
    snd, rcv = H.random_graph(rng, N, E, sort_by=sort_by)
    x, y, s, dm = H.random_operands(rng, N, E, X, Y, S, K, Z, dtype=dtype)
    coef = H.pack_table(idx, val, mix, val_dtype=dtype)
    return dict(idx=idx, val=val, mix=mix, snd=snd, rcv=rcv, x=x, y=y, s=s, dm=dm, coef=coef,
                params=ConvolutionParams(num_out=Z, num_scalars=S))


def _check(p, out, grads, tol=None):
    tol = tol or {}
    ref, mag = H.forward_reference(p["idx"], p["val"], p["mix"], p["x"], p["y"], p["s"], p["snd"], p["rcv"],
                                   p["params"].num_out)
    H.assert_parity(out.detach().cpu().numpy(), ref, mag, "out", **tol)
    refs, mags = H.backward_reference(p["idx"], p["val"], p["mix"], p["x"], p["y"], p["s"], p["snd"],
                                      p["rcv"], p["dm"])
    for g, r, m, name in zip(grads, refs, mags, ("dx", "dy", "ds")):
        H.assert_parity(g.detach().cpu().numpy(), r, m, name, **tol)


@pytest.mark.parametrize("ordering", ["RECEIVER", "NONE"])
@pytest.mark.parametrize("deterministic", [False, True])
def test_autograd_matches_oracle(ordering, deterministic):
    p = _problem(1, sort_by="receiver" if ordering == "RECEIVER" else None)
    x, y, s = (dev(p[k], grad=True) for k in ("x", "y", "s"))
    with e3j_amd.config.use(deterministic=deterministic, debug_level=1):
        out = convolution(p["coef"], x, y, s, dev(p["snd"]), dev(p["rcv"]), p["params"], ordering)
        grads = torch.autograd.grad(out, (x, y, s), dev(p["dm"]))
    _check(p, out, grads)


def test_row_order_does_not_change_results():
    """The locality-aware row order only changes which rows run together: forward bits are identical."""
    p = _problem(12, N=200, E=3000, K=32)
    args = [dev(p[k]) for k in ("x", "y", "s")]
    snd, rcv = dev(p["snd"]), dev(p["rcv"])
    outs = []
    for rounds in (0, 1, 4):
        with e3j_amd.config.use(locality_rounds=rounds):
            outs.append(convolution(p["coef"], *args, snd, rcv, p["params"]))
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])


def test_convolution_bwd_direct_and_deterministic_bits():
    p = _problem(2, N=64, E=2000, K=32)
    args = [dev(p[k]) for k in ("x", "y", "s")]
    snd, rcv, dm = dev(p["snd"]), dev(p["rcv"]), dev(p["dm"])
    with e3j_amd.config.use(deterministic=True):
        base = convolution_bwd(p["coef"], *args, snd, rcv, dm, p["params"])
        for _ in range(5):
            again = convolution_bwd(p["coef"], *args, snd, rcv, dm, p["params"])
            for a, b in zip(base, again):
                assert torch.equal(a, b)
    fast = convolution_bwd(p["coef"], *args, snd, rcv, dm, p["params"])
    out = convolution(p["coef"], *args, snd, rcv, p["params"])
    _check(p, out, fast)
    _check(p, out, base)


@pytest.mark.parametrize("channels", [32, 128])
def test_fifty_runs_give_the_same_bits(channels):
    """The reference's determinism checks (`tests/test_ops/test_convolution_op.py:322-342`: 50
    repeats of the forward and of the gradient, zero tolerance).  The forward is bit-reproducible
    as it stands; the gradient under `config(deterministic=True)` (the default backward adds dx
    with float atomics, in an order that varies)."""
    p = _problem(12, N=200, E=6000, K=channels)
    x, y, s = (dev(p[k], grad=True) for k in ("x", "y", "s"))
    snd, rcv, dm = dev(p["snd"]), dev(p["rcv"]), dev(p["dm"])
    base = convolution(p["coef"], x, y, s, snd, rcv, p["params"])
    for _ in range(50):
        assert torch.equal(base, convolution(p["coef"], x, y, s, snd, rcv, p["params"]))
    with e3j_amd.config.use(deterministic=True):
        def grads():
            out = convolution(p["coef"], x, y, s, snd, rcv, p["params"])
            return torch.autograd.grad(out, (x, y, s), dm)
        first = grads()
        for _ in range(50):
            for a, b in zip(first, grads()):
                assert torch.equal(a, b)
    _check(p, base.detach(), first)


def test_two_dimensional_x_means_one_channel():
    p = _problem(3, K=1)
    x, y, s = dev(p["x"][:, :, 0], grad=True), dev(p["y"], grad=True), dev(p["s"], grad=True)
    out = convolution(p["coef"], x, y, s, dev(p["snd"]), dev(p["rcv"]), p["params"])
    assert out.shape == (p["x"].shape[0], p["params"].num_out)
    grads = torch.autograd.grad(out, (x, y, s), dev(p["dm"][:, :, 0]))
    assert grads[0].shape == x.shape
    _check(p, out.unsqueeze(-1), (grads[0].unsqueeze(-1), grads[1], grads[2]))


def test_leading_layout_and_float64():
    p = _problem(4, dtype=np.float64)
    xl, sl, dml = (np.ascontiguousarray(p[k].swapaxes(1, 2)) for k in ("x", "s", "dm"))
    x, y, s = dev(xl, grad=True), dev(p["y"], grad=True), dev(sl, grad=True)
    out = convolution(p["coef"], x, y, s, dev(p["snd"]), dev(p["rcv"]), p["params"], layout="LEADING_CHANNELS")
    grads = torch.autograd.grad(out, (x, y, s), dev(dml))
    tol = dict(rtol=1e-12, atol=1e-12, ulps=0.0)
    _check(p, out.transpose(1, 2), (grads[0].transpose(1, 2), grads[1], grads[2].transpose(1, 2)), tol)


def _dense_reference(p, x, y, s):
    """Independent torch restatement (dense einsum), differentiable to any order."""
    Z, X, Y = p["params"].num_out, p["x"].shape[1], p["y"].shape[1]
    dense = torch.zeros((Z, X, Y), dtype=x.dtype, device=x.device)
    dense.index_put_(tuple(torch.as_tensor(p["idx"].T, device=x.device)),
                     torch.as_tensor(p["val"], dtype=x.dtype, device=x.device), accumulate=True)
    snd = torch.as_tensor(p["snd"], dtype=torch.long, device=x.device)
    rcv = torch.as_tensor(p["rcv"], dtype=torch.long, device=x.device)
    msg = torch.einsum("ijk,ejc,ek->eic", dense, x[snd], y) * s[:, torch.as_tensor(p["mix"], device=x.device), :]
    return torch.zeros((x.shape[0], Z, x.shape[2]), dtype=x.dtype, device=x.device).index_add(0, rcv, msg)


def test_double_backward_matches_autograd_of_dense_form():
    """Hessian-vector products through convolution_bwd's own backward
    (src/e3j/ops/convolution.py:535-562; tests/test_ops/test_convolution_jax_transforms.py:644-767)."""
    p = _problem(5, N=6, E=20, K=4, dtype=np.float64)
    snd, rcv = dev(p["snd"]), dev(p["rcv"])

    def scalar(fn, x, y, s):
        out = fn(x, y, s)
        g = torch.autograd.grad(out, (x, y, s), dev(p["dm"]), create_graph=True)
        return sum((gi ** 2).sum() for gi in g) + (out ** 3).sum()

    ours = [dev(p[k], grad=True) for k in ("x", "y", "s")]
    theirs = [dev(p[k], grad=True) for k in ("x", "y", "s")]
    a = scalar(lambda x, y, s: convolution(p["coef"], x, y, s, snd, rcv, p["params"]), *ours)
    b = scalar(lambda x, y, s: _dense_reference(p, x, y, s), *theirs)
    torch.testing.assert_close(a, b, rtol=1e-10, atol=1e-10)
    ga = torch.autograd.grad(a, ours)
    gb = torch.autograd.grad(b, theirs)
    for u, v in zip(ga, gb):
        torch.testing.assert_close(u, v, rtol=1e-9, atol=1e-9)


@pytest.mark.parametrize("irreps, l_max, K, layout, unrolled", [
    ("0e+1o", 2, 16, "TRAILING_CHANNELS", False),           # table-driven kernels, signs in the table
    ("0e+1o", 2, 32, "TRAILING_CHANNELS", True),            # unrolled kernels, signs as a y mask
    ("0e+1o+2e+3o", 3, 64, "TRAILING_CHANNELS", True),
    ("0e+1o+2e+3o", 3, 64, "LEADING_CHANNELS", True),
])
def test_sender_ordering_on_symmetric_graph(irreps, l_max, K, layout, unrolled):
    """SENDER ordering = RECEIVER ordering on a symmetric graph with y_ba = p y_ab, s_ba = s_ab
    (tests/test_convolution.py:351-456)."""
    rng = np.random.default_rng(6)
    N = 10
    pos = rng.normal(size=(N, 3))
    pairs = [(a, b) for a in range(N) for b in range(N) if a != b and np.linalg.norm(pos[a] - pos[b]) < 1.6]
    snd = np.array([a for a, b in pairs], dtype=np.int32)
    rcv = np.array([b for a, b in pairs], dtype=np.int32)
    y_irreps = "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(l_max + 1))
    out_irreps = irreps if l_max == 3 else "0e+1o+2e"
    module_r = Convolution((irreps, y_irreps), out_irreps, graph_ordering="RECEIVER", layout=layout)
    module_s = Convolution((irreps, y_irreps), out_irreps, graph_ordering="SENDER", layout=layout)
    vec = torch.from_numpy(pos[snd] - pos[rcv])
    y = Harmonics(l_max, normalize=True)(vec).float().numpy()
    dist = np.linalg.norm(pos[snd] - pos[rcv], axis=-1)
    S = module_r.params.num_scalars
    X = module_r.source[0].dim
    w = rng.normal(size=(S, K)).astype(np.float32)
    s = (np.cos(dist)[:, None, None] * w[None]).astype(np.float32)        # symmetric in (a, b)
    x = rng.normal(size=(N, X, K)).astype(np.float32)
    dm = rng.normal(size=(N, module_r.target.dim, K)).astype(np.float32)
    if layout == "LEADING_CHANNELS":
        s, x, dm = (np.ascontiguousarray(t.transpose(0, 2, 1)) for t in (s, x, dm))
    # which kernels serve the signed table of the SENDER ordering
    from e3j_amd.ops import _Table
    c = module_s.coef
    signed = e3j_amd.Coef4D(c.val * module_s.y_parity[c.idx[:, 2].astype(np.int64)], c.idx, "float32",
                            c.idx_dtype).pack()
    sig, _, flip = _Table.get(signed, np.float32).signature((X, y.shape[1], module_s.target.dim, S), K,
                                                            module_s.layout)
    assert (sig >= 0 and flip != 0) == unrolled

    def run(module, order):
        xs, ys, ss = dev(x, grad=True), dev(y[order], grad=True), dev(s[order], grad=True)
        out = module(xs, ys, ss, dev(snd[order]), dev(rcv[order]))
        gx, gy, gs = torch.autograd.grad(out, (xs, ys, ss), dev(dm))
        inverse = np.argsort(order)
        return out, gx, gy[inverse], gs[inverse]

    by_receiver = run(module_r, np.argsort(rcv, kind="stable"))
    by_sender = run(module_s, np.argsort(snd, kind="stable"))
    for a, b in zip(by_receiver, by_sender):
        torch.testing.assert_close(a, b, rtol=2e-5, atol=2e-5)


def test_batched_graphs_fold_with_padding():
    """A batch of padded graphs folded into one graph equals a loop over the graphs
    (tests/test_ops/test_convolution_jax_transforms.py:197-226)."""
    B, p = 3, _problem(7, N=8, E=30)
    rng = np.random.default_rng(8)
    xs = rng.normal(size=(B,) + p["x"].shape).astype(np.float32)
    ys = rng.normal(size=(B,) + p["y"].shape).astype(np.float32)
    ss = rng.normal(size=(B,) + p["s"].shape).astype(np.float32)
    snd = np.stack([p["snd"]] * B)
    rcv = np.stack([p["rcv"]] * B)
    for b in range(B):                          # tail padding of different lengths per graph
        snd[b, 30 - 2 * (b + 1):] = O.DUMMY_INDEX
        rcv[b, 30 - 2 * (b + 1):] = O.DUMMY_INDEX
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        out = e3j_amd.convolution_batched(p["coef"], dev(xs), dev(ys), dev(ss), dev(snd), dev(rcv), p["params"])
    assert any(issubclass(w.category, e3j_amd.ConvolutionBatchingWarning) for w in caught)
    for b in range(B):
        ref, mag = H.forward_reference(p["idx"], p["val"], p["mix"], xs[b], ys[b], ss[b], snd[b], rcv[b],
                                       p["params"].num_out)
        H.assert_parity(out[b].cpu().numpy(), ref, mag, f"graph {b}")
    shared = e3j_amd.convolution_batched(p["coef"], dev(xs), dev(ys), dev(ss), dev(p["snd"]), dev(p["rcv"]),
                                         p["params"])
    ref, mag = H.forward_reference(p["idx"], p["val"], p["mix"], xs[1], ys[1], ss[1], p["snd"], p["rcv"],
                                   p["params"].num_out)
    H.assert_parity(shared[1].cpu().numpy(), ref, mag, "shared graph")


# --- module level -----------------------------------------------------------------------
def _wigner_d(space, rot):
    from tests.test_host_logic import _wigner_d as one
    blocks = [one(ir.l, rot) * (ir.p ** 0) for mul, ir in space for _ in range(mul)]
    dim = sum(b.shape[0] for b in blocks)
    out, at = np.zeros((dim, dim)), 0
    for b in blocks:
        out[at:at + b.shape[0], at:at + b.shape[0]] = b
        at += b.shape[0]
    return out


def test_module_is_equivariant_and_shapes():
    """Rotating node features and edge harmonics rotates the messages (tests/test_convolution.py:112-167)."""
    from scipy.spatial.transform import Rotation
    rng = np.random.default_rng(9)
    N, E, K = 7, 40, 8
    module = Convolution(("0e+1o+2e", "0e+1o+2e"), "0e+1o+2e", graph_ordering="RECEIVER", avg_num_neighbors=5.0)
    snd, rcv = H.random_graph(rng, N, E)
    vec = rng.normal(size=(E, 3))
    rot = Rotation.from_rotvec([0.4, 0.2, -0.9]).as_matrix()
    sh = Harmonics(2, normalize=True)
    x = rng.normal(size=(N, module.source[0].dim, K))
    s = rng.normal(size=(E, module.params.num_scalars, K))
    d_x, d_out = _wigner_d(module.source[0], rot), _wigner_d(module.target, rot)

    def run(x_, vec_):
        y_ = sh(torch.from_numpy(vec_)).cuda()
        return module(dev(x_), y_, dev(s), dev(snd), dev(rcv)).cpu().numpy()

    out = run(x, vec)
    assert out.shape == (N, module.target.dim, K)
    out_rot = run(np.einsum("ij,njc->nic", d_x, x), vec @ rot.T)
    # coefficient values are stored as float32 (like the reference's tables): equivariance holds to that rounding
    np.testing.assert_allclose(out_rot, np.einsum("ij,njc->nic", d_out, out), rtol=0, atol=5e-6)


def test_module_node_mask_and_dtype_promotion():
    w_name = "0e+1o"
    module = Convolution((w_name, "0e+1o"), None, graph_ordering="RECEIVER")
    rng = np.random.default_rng(10)
    N, E, K = 6, 24, 4
    # padding nodes (4, 5) lie at the tail and padding edges only connect padding nodes, as the
    # reference requires (src/e3j/core/convolution.py:367-372): they form the tail of the sorted list
    rcv = np.sort(np.concatenate([rng.integers(0, 4, E - 6), rng.integers(4, 6, 6)])).astype(np.int32)
    snd = np.where(rcv < 4, rng.integers(0, 4, E), rng.integers(4, 6, E)).astype(np.int32)
    x = rng.normal(size=(N, 4, K)).astype(np.float32)
    y = rng.normal(size=(E, 4)).astype(np.float32)
    s = rng.normal(size=(E, module.params.num_scalars, K)).astype(np.float32)
    mask = np.arange(N) < 4
    out = module(dev(x), dev(y), dev(s), dev(snd), dev(rcv), node_mask=dev(mask))
    keep = (snd < 4) & (rcv < 4)
    ref = module(dev(x), dev(y[keep]), dev(s[keep]), dev(snd[keep]), dev(rcv[keep]))
    torch.testing.assert_close(out, ref, rtol=1e-6, atol=1e-6)
    assert not out[4:].any()
    assert module(dev(x.astype(np.float64)), dev(y), dev(s), dev(snd), dev(rcv)).dtype == torch.float64


# --- errors of the reference's operator ------------------------------------------------
def test_operator_errors():
    p = _problem(11)
    x, y, s, snd, rcv = (dev(p[k]) for k in ("x", "y", "s", "snd", "rcv"))
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        convolution(p["coef"], x.cpu(), y, s, snd, rcv, p["params"])
    with pytest.raises(NotImplementedError, match="only one channel"):
        convolution(p["coef"], x, torch.stack([y, y], -1), s, snd, rcv, p["params"])
    with pytest.raises(TypeError, match="concrete"):
        convolution(torch.from_numpy(p["coef"]), x, y, s, snd, rcv, p["params"])
    with pytest.raises(ValueError, match="y_parity"):
        convolution(p["coef"], x, y, s, snd, rcv, p["params"], GraphOrdering.SENDER)
    with pytest.raises(TypeError, match="Cast the operands"):
        convolution(p["coef"], x.bfloat16(), y.bfloat16(), s.bfloat16(), snd, rcv, p["params"])


def test_opt_in_cache_reuses_per_index_tensor_pair_and_follows_in_place_changes():
    import e3j_amd
    from e3j_amd import ops
    p = _problem(8, N=20, E=200, K=16)
    x, y, s = (dev(p[k]) for k in ("x", "y", "s"))
    snd, rcv = dev(p["snd"]), dev(p["rcv"])
    ops.clear_graph_cache()
    convolution(p["coef"], x, y, s, snd, rcv, p["params"])
    assert len(ops._GRAPH_CACHE) == 0                      # off unless asked for
    with e3j_amd.config.use(graph_cache=True):
        first = convolution(p["coef"], x, y, s, snd, rcv, p["params"])
        assert len(ops._GRAPH_CACHE) == 1
        again = convolution(p["coef"], x, y, s, snd, rcv, p["params"])
        assert len(ops._GRAPH_CACHE) == 1 and torch.equal(first, again)
        # an in-place change of the senders through torch must not be served from the cache
        snd[:] = torch.roll(snd, 1)
        changed = convolution(p["coef"], x, y, s, snd, rcv, p["params"])
        ref, mag = H.forward_reference(p["idx"], p["val"], p["mix"], p["x"], p["y"], p["s"],
                                       np.roll(p["snd"], 1), p["rcv"], p["params"].num_out)
        H.assert_parity(changed.cpu().numpy(), ref, mag, "after in-place change")
        del snd, rcv
        import gc
        gc.collect()
        assert len(ops._GRAPH_CACHE) == 0                  # entries die with their tensors


def test_index_buffer_rewritten_behind_the_version_counter():
    """A neighbour list rewritten through `.data` (or a raw pointer) keeps its version counter: the
    default path prepares the adjacency on every call and follows the new contents; a
    `prepare_graph` handle is rebuilt by its owner."""
    from e3j_amd import prepare_graph
    p = _problem(9, N=24, E=240, K=16)
    x, y, s = (dev(p[k], grad=True) for k in ("x", "y", "s"))
    snd, rcv = dev(p["snd"]), dev(p["rcv"])
    dm = dev(p["dm"])

    def check(out, grads, senders, what):
        ref, mag = H.forward_reference(p["idx"], p["val"], p["mix"], p["x"], p["y"], p["s"], senders, p["rcv"],
                                       p["params"].num_out)
        H.assert_parity(out.detach().cpu().numpy(), ref, mag, what + " out")
        refs, mags = H.backward_reference(p["idx"], p["val"], p["mix"], p["x"], p["y"], p["s"], senders, p["rcv"],
                                          p["dm"])
        for g, r, m, name in zip(grads, refs, mags, ("dx", "dy", "ds")):
            H.assert_parity(g.cpu().numpy(), r, m, f"{what} {name}")

    out = convolution(p["coef"], x, y, s, snd, rcv, p["params"])
    check(out, torch.autograd.grad(out, (x, y, s), dm), p["snd"], "before")
    version = snd._version
    rolled = np.roll(p["snd"], 3)
    snd.data.copy_(torch.as_tensor(rolled))                # rewritten behind the version counter
    assert snd._version == version
    out = convolution(p["coef"], x, y, s, snd, rcv, p["params"])
    check(out, torch.autograd.grad(out, (x, y, s), dm), rolled, "after the rewrite")
    # the explicit handle: one preparation for forward and backward of several calls
    handle = prepare_graph(snd, rcv, 24)
    for _ in range(2):
        out = convolution(p["coef"], x, y, s, snd, rcv, p["params"], graph=handle)
        check(out, torch.autograd.grad(out, (x, y, s), dm), rolled, "with a handle")
    with pytest.raises(ValueError, match="prepared for"):
        convolution(p["coef"], x, y[:-1], s[:-1], snd[:-1], rcv[:-1], p["params"], graph=handle)


def test_prepared_graph_used_on_another_stream_waits_for_its_preparation():
    from e3j_amd import prepare_graph
    p = _problem(10, N=2000, E=60000, K=16)
    x, y, s = (dev(p[k]) for k in ("x", "y", "s"))
    snd, rcv = dev(p["snd"]), dev(p["rcv"])
    want = convolution(p["coef"], x, y, s, snd, rcv, p["params"])
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    handle = prepare_graph(snd, rcv, 2000)                 # prepared on the current stream, not waited for
    with torch.cuda.stream(side):
        got = convolution(p["coef"], x, y, s, snd, rcv, p["params"], graph=handle)
    side.synchronize()
    assert torch.equal(got, want)


def test_tables_without_an_unrolled_kernel_warn_once():
    p = _problem(9, N=10, E=60, K=8)
    x, y, s = (dev(p[k]) for k in ("x", "y", "s"))
    snd, rcv = dev(p["snd"]), dev(p["rcv"])
    with warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter("always")
        convolution(p["coef"], x, y, s, snd, rcv, p["params"])
        convolution(p["coef"], x, y, s, snd, rcv, p["params"])
    hits = [w for w in seen if issubclass(w.category, e3j_amd.TableDrivenKernelWarning)]
    assert len(hits) == 1 and "jit" in str(hits[0].message)


def test_third_order_gradients_match_autograd_of_dense_form():
    """Differentiable to any reverse-mode order
    (tests/test_ops/test_convolution_jax_transforms.py:713-767)."""
    p = _problem(15, N=5, E=14, K=2, X=3, Y=4, Z=5, S=3, nnz=30, dtype=np.float64)
    snd, rcv = dev(p["snd"]), dev(p["rcv"])

    def third(fn):
        x, y, s = (dev(p[k], grad=True) for k in ("x", "y", "s"))
        out = fn(x, y, s)
        g1 = torch.autograd.grad((out ** 2).sum(), (x, y, s), create_graph=True)
        g2 = torch.autograd.grad(sum((g ** 2).sum() for g in g1), (x, y, s), create_graph=True)
        return torch.autograd.grad(sum((g ** 2).sum() for g in g2), (x, y, s))

    ours = third(lambda x, y, s: convolution(p["coef"], x, y, s, snd, rcv, p["params"]))
    theirs = third(lambda x, y, s: _dense_reference(p, x, y, s))
    for u, v in zip(ours, theirs):
        torch.testing.assert_close(u, v, rtol=1e-8, atol=1e-8 * float(v.abs().max()))


def test_torch_func_transforms():
    """vmap (operands batched, graph shared or batched), Jacobians, Hessian-vector products and
    per-sample gradients through `torch.func`; forward mode raises
    (tests/test_ops/test_convolution_jax_transforms.py:108-196,622-711,770-788,843-900)."""
    from torch.func import grad, jacrev, vmap
    p = _problem(16, N=6, E=20, K=4, dtype=np.float64)
    snd, rcv = dev(p["snd"]), dev(p["rcv"])
    f = lambda x, y, s: convolution(p["coef"], x, y, s, snd, rcv, p["params"])  # noqa: E731
    dense = lambda x, y, s: _dense_reference(p, x, y, s)  # noqa: E731
    rng = np.random.default_rng(17)
    B = 3
    xb, yb, sb = (dev(rng.normal(size=(B,) + p[k].shape)) for k in ("x", "y", "s"))
    want = torch.stack([dense(xb[b], yb[b], sb[b]) for b in range(B)])
    torch.testing.assert_close(vmap(f)(xb, yb, sb), want)
    # only x batched: the other operands are broadcast over the batch
    torch.testing.assert_close(vmap(f, in_dims=(0, None, None))(xb, yb[0], sb[0]),
                               torch.stack([dense(xb[b], yb[0], sb[0]) for b in range(B)]))
    # a graph per batch entry: folded into one disjoint graph, with the reference's warning
    graphs = [H.random_graph(rng, 6, 20) for _ in range(B)]
    snd_b = dev(np.stack([g[0] for g in graphs]))
    rcv_b = dev(np.stack([g[1] for g in graphs]))
    g_fn = lambda x, y, s, a, b: convolution(p["coef"], x, y, s, a, b, p["params"])  # noqa: E731
    with pytest.warns(e3j_amd.ConvolutionBatchingWarning):
        got = vmap(g_fn)(xb, yb, sb, snd_b, rcv_b)
    for b in range(B):
        q = dict(p, snd=graphs[b][0], rcv=graphs[b][1])
        torch.testing.assert_close(got[b], _dense_reference(q, xb[b], yb[b], sb[b]))
    # per-sample gradients and a Jacobian (vmap over the backward operator)
    w = dev(rng.normal(size=p["dm"].shape))
    energy = lambda fn: (lambda x, y, s: (fn(x, y, s) * w).sum())  # noqa: E731
    ours = vmap(grad(energy(f), argnums=(0, 1, 2)))(xb, yb, sb)
    theirs = vmap(grad(energy(dense), argnums=(0, 1, 2)))(xb, yb, sb)
    for u, v in zip(ours, theirs):
        torch.testing.assert_close(u, v)
    x0, y0, s0 = xb[0], yb[0], sb[0]
    torch.testing.assert_close(jacrev(f, argnums=1)(x0, y0, s0), jacrev(dense, argnums=1)(x0, y0, s0))
    # Hessian-vector product under vmap
    hvp = lambda fn: (lambda x, y, s: grad(lambda a: (grad(energy(fn))(a, y, s) * x).sum())(x))  # noqa: E731
    torch.testing.assert_close(vmap(hvp(f))(xb, yb, sb), vmap(hvp(dense))(xb, yb, sb))
    with pytest.raises(RuntimeError):   # forward-mode differentiation is not defined for the operator
        torch.func.jvp(f, (x0, y0, s0), (x0, y0, s0))


@pytest.mark.parametrize("layout", ["TRAILING_CHANNELS", "LEADING_CHANNELS"])
@pytest.mark.parametrize("ordering", ["RECEIVER", "NONE"])
def test_float16_operands(layout, ordering):
    """float16 values run the table-driven kernels in half precision
    (tests/test_ops/test_dtype.py:253-330): parity with the float64 checker on the rounded
    operands, within the rounding of a half-precision running sum."""
    p = _problem(18, N=15, E=90, K=24, nnz=50, sort_by="receiver" if ordering == "RECEIVER" else None)
    half = {k: p[k].astype(np.float16) for k in ("x", "y", "s", "dm")}
    val16 = p["val"].astype(np.float16)
    coef = H.pack_table(p["idx"], val16, p["mix"], val_dtype=np.float16)
    lead = layout == "LEADING_CHANNELS"
    t = (lambda a: np.ascontiguousarray(a.transpose(0, 2, 1))) if lead else (lambda a: a)
    back = (lambda g: g.transpose(1, 2)) if lead else (lambda g: g)
    x, y, s = dev(t(half["x"]), grad=True), dev(half["y"], grad=True), dev(t(half["s"]), grad=True)
    out = convolution(coef, x, y, s, dev(p["snd"]), dev(p["rcv"]), p["params"], ordering, layout=layout)
    assert out.dtype == torch.float16
    grads = torch.autograd.grad(out, (x, y, s), dev(t(half["dm"])))
    f64 = {k: v.astype(np.float64) for k, v in half.items()}
    ref, mag = H.forward_reference(p["idx"], val16.astype(np.float64), p["mix"], f64["x"], f64["y"], f64["s"],
                                   p["snd"], p["rcv"], p["params"].num_out)
    refs, mags = H.backward_reference(p["idx"], val16.astype(np.float64), p["mix"], f64["x"], f64["y"], f64["s"],
                                      p["snd"], p["rcv"], f64["dm"])
    eps = 2.0 ** -10
    for got, r, m, name in [(out, ref, mag, "out")] + list(zip(grads, refs, mags, ("dx", "dy", "ds"))):
        got = back(got) if got.dim() == 3 else got
        err = np.abs(got.detach().float().cpu().numpy().astype(np.float64) - r)
        assert np.all(err <= 6 * eps * m + 1e-3), f"{name}: {err.max()} against magnitude {m.max()}"
