"""Synthetic inputs of the benchmark configurations (seeded).

Atoms at uniformly random positions in a cubic box, a radius graph with a 5
Angstrom cutoff (periodic boxes use the minimum image), spherical harmonics of
the unit edge vectors as `y`, normal node features and per-edge per-path radial
weights of variance `1/fan_in`.  Positions and graphs always come from
`numpy.random.default_rng(seed)`.  The large value arrays come from the same
generator when the workload is built on the host, and from a seeded
`torch.Generator` of the device when it is built in GPU memory (the 1M-edge
configuration holds 11 GB of radial weights; drawing them on the host and
copying them would take minutes).
"""

from __future__ import annotations

import dataclasses
import math

import numpy as np
import torch

from .channel_mix import ChannelMix
from .convolution import Convolution
from .edge_features import edge_features
from .harmonics import Harmonics
from .options import Layout
from .radial import radial_linear, supported as radial_supported


@dataclasses.dataclass
class Workload:
    name: str
    module: Convolution
    x: torch.Tensor         # (N, X, K); (N, K, X) in the leading-channels layout
    y: torch.Tensor         # (E, Y)
    s: torch.Tensor         # (E, S, K); (E, K, S)
    dm: torch.Tensor        # (N, Z, K); (N, K, Z)
    sender: torch.Tensor    # (E,) int32
    receiver: torch.Tensor  # (E,) int32
    positions: np.ndarray
    box: float

    @property
    def leading(self) -> bool:
        return self.module.layout == Layout.LEADING_CHANNELS

    def with_layout(self, layout) -> "Workload":
        """The same values in the other memory layout (a module of that layout, axes swapped)."""
        layout = Layout.parse(layout)
        if layout == self.module.layout:
            return self
        m = self.module
        out_filter = "+".join(dict.fromkeys(f"{ir.l}{'e' if ir.p == 1 else 'o'}" for _, ir in m.target))
        module = Convolution((m.source[0], m.source[1]), out_filter, graph_ordering=m.graph_ordering,
                             layout=layout, avg_num_neighbors=m.avg_num_neighbors,
                             normalization=m.normalization)
        swap = {f: getattr(self, f).transpose(1, 2).contiguous() for f in ("x", "s", "dm")}
        return dataclasses.replace(self, module=module, **swap)

    def to(self, device) -> "Workload":
        return dataclasses.replace(self, **{f: getattr(self, f).to(device) for f in
                                            ("x", "y", "s", "dm", "sender", "receiver")})

    def numpy(self) -> dict:
        """Host copies of the operands in the trailing-channels layout, for the CPU checker."""
        w = self.with_layout(Layout.TRAILING_CHANNELS)
        return {f: getattr(w, f).cpu().numpy() for f in ("x", "y", "s", "dm", "sender", "receiver")}

    def table(self):
        """`(idx (nnz, 3), val, mix_idx)` of the module's coefficient table."""
        c = self.module.coef
        idx = np.asarray(c.idx, dtype=np.int64)
        mix = np.zeros(self.module.target.dim, dtype=np.int64)
        mix[idx[:, 0]] = idx[:, 3]
        return idx[:, :3], np.asarray(c.val, dtype=np.float32), self.module._mix.mix_indices

    def head(self, num_receivers: int) -> "Workload":
        """Sub-problem of the first `num_receivers` receivers' edges (receiver-sorted workloads).

        Senders keep their global indices, so `x` is kept whole.
        """
        e = int((self.receiver < num_receivers).sum().item())
        return dataclasses.replace(self, s=self.s[:e], y=self.y[:e], sender=self.sender[:e],
                                   receiver=self.receiver[:e])

    @property
    def num_nodes(self) -> int:
        return int(self.x.shape[0])

    @property
    def num_edges(self) -> int:
        return int(self.y.shape[0])

    @property
    def channels(self) -> int:
        return int(self.x.shape[1 if self.leading else 2])

    def algorithmic_bytes(self, sorted_edges: bool = True) -> dict:
        """Compulsory traffic: each operand element read once, each result written once."""
        n, e, k = self.num_nodes, self.num_edges, self.channels
        d = 2 if self.leading else 1
        X, Y, S, Z = int(self.x.shape[d]), int(self.y.shape[1]), int(self.s.shape[d]), int(self.dm.shape[d])
        fwd = 4 * (n * X * k + e * Y + e * S * k + n * Z * k) + 4 * (e + n + 1)
        bwd = 4 * (2 * n * X * k + 2 * e * Y + 2 * e * S * k + n * Z * k) + 4 * (2 * e + n + 1)
        if not sorted_edges:
            fwd += 4 * e
            bwd += 4 * e
        return {"fwd": fwd, "bwd": bwd, "fwd_bwd": fwd + bwd}


def periodic_box_length(num_atoms: int, neighbours: float, cutoff: float) -> float:
    """Edge of the cube whose density gives `neighbours` atoms within `cutoff`."""
    density = neighbours / (4.0 / 3.0 * math.pi * cutoff ** 3)
    return (num_atoms / density) ** (1.0 / 3.0)


def radius_graph(positions: np.ndarray, cutoff: float, box: float | None):
    """Directed edges `(sender, receiver)` with `|r_s - r_r| < cutoff`, and the vectors r_s - r_r.

    `box`: edge of the periodic cube (minimum image) or None for an open box.
    Edges come out sorted by receiver, then sender.
    """
    from scipy.spatial import cKDTree
    pos = np.asarray(positions, dtype=np.float64)
    if box is not None:
        pos = np.mod(pos, box)
        tree = cKDTree(pos, boxsize=box)
    else:
        tree = cKDTree(pos)
    pairs = tree.query_pairs(cutoff, output_type="ndarray")
    a = np.concatenate([pairs[:, 0], pairs[:, 1]])
    b = np.concatenate([pairs[:, 1], pairs[:, 0]])
    order = np.lexsort((a, b))
    sender, receiver = a[order], b[order]
    vec = pos[sender] - pos[receiver]
    if box is not None:
        vec -= box * np.round(vec / box)
    return sender.astype(np.int32), receiver.astype(np.int32), vec


def path_fan_in(module: Convolution) -> np.ndarray:
    """Number of (x irrep, y irrep) paths feeding each output irrep, per path."""
    degrees = []
    for mul, ir in module.target:
        degrees += [(ir.l, ir.p)] * mul
    counts = {d: degrees.count(d) for d in set(degrees)}
    return np.array([counts[d] for d in degrees], dtype=np.float64)


def _harmonics(vec: np.ndarray, l_max: int, device) -> torch.Tensor:
    unit = torch.from_numpy(vec / np.linalg.norm(vec, axis=-1, keepdims=True)).to(device)
    return Harmonics(l_max, normalization="component")(unit).to(torch.float32)


def _normal(shape, seed: int, device) -> torch.Tensor:
    device = torch.device(device)
    if device.type == "cpu":
        return torch.from_numpy(np.random.default_rng(seed).standard_normal(shape, dtype=np.float32))
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    return torch.randn(shape, dtype=torch.float32, device=device, generator=gen)


def morton_order(positions: np.ndarray, box: float, bits: int = 10) -> np.ndarray:
    """Permutation sorting points along a Z-order curve (atoms numbered coherently in space)."""
    cells = np.clip((positions / box * (1 << bits)).astype(np.int64), 0, (1 << bits) - 1)
    code = np.zeros(len(positions), dtype=np.int64)
    for b in range(bits):
        for axis in range(3):
            code |= ((cells[:, axis] >> b) & 1) << (3 * b + axis)
    return np.argsort(code, kind="stable")


def make_workload(name: str, num_atoms: int, x_irreps: str, l_max: int, out_irreps: str,
                  channels: int, seeds: tuple, *, neighbours: float | None = 30.0,
                  box: float | None = None, periodic: bool = True, cutoff: float = 5.0,
                  device="cpu", spatial_sort: bool = False) -> Workload:
    seed_pos, seed_x, seed_s, seed_dm = seeds
    if box is None:
        box = periodic_box_length(num_atoms, neighbours, cutoff)
    pos = np.random.default_rng(seed_pos).uniform(0.0, box, size=(num_atoms, 3))
    if spatial_sort:  # same atoms, numbered along a space-filling curve instead of at random
        pos = pos[morton_order(pos, box)]
    sender, receiver, vec = radius_graph(pos, cutoff, box if periodic else None)
    y_irreps = "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(l_max + 1))
    module = Convolution((x_irreps, y_irreps), out_irreps, graph_ordering="RECEIVER")
    X, Z, S = module.source[0].dim, module.target.dim, module.params.num_scalars
    E = sender.shape[0]
    x = _normal((num_atoms, X, channels), seed_x, device)
    y = _harmonics(vec, l_max, device)
    std = torch.from_numpy((1.0 / np.sqrt(path_fan_in(module))).astype(np.float32)).to(device)
    s = _normal((E, S, channels), seed_s, device)
    s *= std[None, :, None]
    dm = _normal((num_atoms, Z, channels), seed_dm, device)
    return Workload(name, module, x, y, s, dm, torch.from_numpy(sender).to(device),
                    torch.from_numpy(receiver).to(device), pos, box)


def config1(scale: float = 1.0, device="cpu") -> Workload:
    """1 000 atoms in an open 20 A box, 32 channels, 0e+1o x lmax 2 -> 0e+1o+2e."""
    n = max(8, int(1000 * scale))
    return make_workload("cfg1", n, "0e+1o", 2, "0e+1o+2e", 32, (1, 2, 3, 4),
                         box=20.0 * scale ** (1.0 / 3.0), periodic=False, device=device)


def config2(scale: float = 1.0, out_irreps: str = "0e+1o+2e", channels: int = 64, device="cpu") -> Workload:
    """5 000 atoms, ~30 neighbours (~150k edges), 64 channels, 0e+1o+2e x lmax 3."""
    n = max(8, int(5000 * scale))
    return make_workload("cfg2", n, "0e+1o+2e", 3, out_irreps, channels, (11, 12, 13, 14), device=device)


def config3(scale: float = 1.0, channels: int = 128, device="cpu", spatial_sort: bool = False) -> Workload:
    """32 000 atoms, ~30 neighbours (~1M edges), 128 channels, 0e..3o x lmax 3 -> 0e..3o."""
    n = max(8, int(32000 * scale))
    return make_workload("cfg3", n, "0e+1o+2e+3o", 3, "0e+1o+2e+3o", channels, (21, 22, 23, 24),
                         device=device, spatial_sort=spatial_sort)


def config4(scale: float = 1.0, device="cpu") -> Workload:
    """Shapes of config 2 with a skewed degree distribution and edges in random order.

    10 % of the atoms (hubs) receive about 120 edges drawn from a pool of 40 % of the
    atoms, the rest about 20; edge vectors are random unit vectors.
    """
    n = max(40, int(5000 * scale))
    rng = np.random.default_rng(31)
    hubs = rng.permutation(n)[: n // 10]
    pool = rng.permutation(n)[: max(4, (4 * n) // 10)]
    is_hub = np.zeros(n, dtype=bool)
    is_hub[hubs] = True
    degree = np.where(is_hub, rng.poisson(120, n), rng.poisson(20, n))
    receiver = np.repeat(np.arange(n), degree)
    sender = np.where(is_hub[receiver], pool[rng.integers(0, pool.shape[0], receiver.shape[0])],
                      rng.integers(0, n, receiver.shape[0]))
    shuffle = np.random.default_rng(32).permutation(receiver.shape[0])
    sender, receiver = sender[shuffle].astype(np.int32), receiver[shuffle].astype(np.int32)
    vec = np.random.default_rng(33).standard_normal((receiver.shape[0], 3))
    module = Convolution(("0e+1o+2e", "0e+1o+2e+3o"), "0e+1o+2e", graph_ordering="NONE")
    X, Z, S = module.source[0].dim, module.target.dim, module.params.num_scalars
    E = sender.shape[0]
    x = _normal((n, X, 64), 34, device)
    y = _harmonics(vec, 3, device)
    std = torch.from_numpy((1.0 / np.sqrt(path_fan_in(module))).astype(np.float32)).to(device)
    s = _normal((E, S, 64), 35, device) * std[None, :, None]
    dm = _normal((n, Z, 64), 36, device)
    return Workload("cfg4", module, x, y, s, dm, torch.from_numpy(sender).to(device),
                    torch.from_numpy(receiver).to(device), np.zeros((n, 3)), 0.0)


class EnergyModel:
    """Two stacked convolutions with per-degree channel mixing and a scalar energy readout.

    The layer sequence of the end-to-end configuration: positions -> edge vectors ->
    (spherical harmonics, Bessel radial basis -> MLP -> per-path radial weights) ->
    Convolution -> Linear mixing, twice, then a linear readout on the `0e` rows summed over
    the atoms.  Everything but the convolution is plain tensor arithmetic, so the gradient
    with respect to the positions reaches the fused kernels' VJPs through `y` and `s`
    (layer 2 also through `x`).  `convolve(layer, x, y, s, sender, receiver)` can be
    replaced to evaluate the same model with another implementation of the operator.
    """

    def __init__(self, channels: int = 64, irreps: str = "0e+1o+2e+3o", l_max: int = 3,
                 num_basis: int = 8, hidden: int = 32, cutoff: float = 5.0,
                 avg_num_neighbors: float = 30.0, seeds=(43, 44, 45)):
        y_irreps = "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(l_max + 1))
        self.layers = [Convolution((irreps, y_irreps), irreps, graph_ordering="RECEIVER",
                                   avg_num_neighbors=avg_num_neighbors) for _ in range(2)]
        self.channels, self.cutoff, self.num_basis = channels, float(cutoff), num_basis
        self.harmonics = Harmonics(l_max, normalization="component")
        module = self.layers[0]
        self.num_x, self.num_paths = module.source[0].dim, module.params.num_scalars
        # (degree block of the output, copies, components) in row order
        self.blocks = [(mul, 2 * ir.l + 1) for mul, ir in module.target]
        seed_mlp, seed_mix, seed_read = seeds
        rng = np.random.default_rng(seed_mlp)
        self.mlp = [(rng.standard_normal((num_basis, hidden)) / math.sqrt(num_basis),
                     rng.standard_normal((hidden, self.num_paths * channels)) / math.sqrt(hidden))
                    for _ in self.layers]
        rng = np.random.default_rng(seed_mix)
        self.mix = [[rng.standard_normal((mul, channels, channels)) / math.sqrt(mul * channels)
                     for mul, _ in self.blocks] for _ in self.layers]
        self.readout = np.random.default_rng(seed_read).standard_normal(channels) / math.sqrt(channels)
        self._weights: dict = {}

    def _t(self, array, like: torch.Tensor) -> torch.Tensor:
        """A weight array as a tensor beside `like`; uploaded once per dtype and device."""
        key = (id(array), like.dtype, like.device)
        hit = self._weights.get(key)
        if hit is None:
            hit = self._weights[key] = torch.as_tensor(array, dtype=like.dtype, device=like.device)
        return hit

    def radial_basis(self, r: torch.Tensor) -> torch.Tensor:
        """Bessel functions `sqrt(2/rc) sin(n pi r / rc) / r` times a smooth cutoff envelope."""
        n = torch.arange(1, self.num_basis + 1, dtype=r.dtype, device=r.device)
        u = (r / self.cutoff).clamp(max=1.0)
        envelope = 1.0 - 10.0 * u ** 3 + 15.0 * u ** 4 - 6.0 * u ** 5
        bessel = math.sqrt(2.0 / self.cutoff) * torch.sin(n * math.pi * r[:, None] / self.cutoff) / r[:, None]
        return bessel * envelope[:, None]

    def edge_inputs(self, positions, sender, receiver, shift):
        vec = positions[sender.long()] - positions[receiver.long()] + shift
        r = torch.linalg.vector_norm(vec, dim=-1)
        return self.harmonics(vec / r[:, None]), self.radial_basis(r)

    def convolve(self, layer, x, y, s, sender, receiver):
        # one adjacency for all layers of a step
        held = getattr(self, "_prepared", None)
        if x.is_cuda and (held is None or held[0] is not sender or held[1] is not receiver):
            from .ops import prepare_graph
            # (rebuilt for every step here: pairing the rows would not pay for itself)
            held = self._prepared = (sender, receiver, prepare_graph(sender, receiver, x.shape[0],
                                                                     self.layers[layer].graph_ordering,
                                                                     pair_rows=False))
        return self.layers[layer](x, y, s, sender, receiver, graph=held[2] if x.is_cuda else None)

    def energy(self, positions, node_features, sender, receiver, shift, convolve=None):
        """Scalar energy.  On the GPU (and with the library's own convolution) the steps around the
        convolutions are kernels of the library as well: one launch from positions to harmonics and
        hidden radial layers (`edge_features`), the matrix-core product for the radial weights
        (`radial_linear`), one regrouping launch either side of the mixing products (`ChannelMix`).
        Anywhere else (host tensors, a replaced `convolve`) the same formulas run as tensor
        operations: that form is what the tests differentiate on the host."""
        kernels = positions.is_cuda and convolve is None
        convolve = convolve or self.convolve
        self._prepared = None   # the neighbour list may have been rewritten in place since the last step
        if kernels:
            w1 = self._stacked_w1(positions)
            y, hidden_layers = edge_features(positions, sender, receiver, shift, w1, max(self.harmonics.degrees),
                                             self.cutoff, self.harmonics.normalization)
            hidden_layers = hidden_layers.unbind(0)
        else:
            y, basis = self.edge_inputs(positions, sender, receiver, shift)
        x = node_features
        for layer, (w1, w2) in enumerate(self.mlp):
            hidden = hidden_layers[layer] if kernels else torch.nn.functional.silu(basis @ self._t(w1, basis))
            last = self._t(w2, hidden)
            # the weights of every path and channel: the matrix-core kernel where it applies
            s = radial_linear(hidden, last) if radial_supported(hidden, last) else hidden @ last
            s = s.reshape(-1, self.num_paths, self.channels)
            out = convolve(layer, x, y, s, sender, receiver)          # (N, Z, K)
            if kernels:
                x = self._mixer(layer)(out)
                continue
            rows, mixed = 0, []
            for (mul, dim), w in zip(self.blocks, self.mix[layer]):
                block = out[:, rows:rows + mul * dim, :].reshape(-1, mul, dim, self.channels)
                mixed.append(torch.einsum("numk,ukc->nmc", block, self._t(w, out)))
                rows += mul * dim
            x = torch.cat(mixed, dim=1)                                # (N, X, K)
        return (x[:, 0, :] @ self._t(self.readout, x)).sum()

    def _stacked_w1(self, like: torch.Tensor) -> torch.Tensor:
        """First layers of the radial networks of all convolution layers, `(layers, num_basis, hidden)`."""
        key = ("w1", like.dtype, like.device)
        hit = self._weights.get(key)
        if hit is None:
            hit = self._weights[key] = torch.as_tensor(np.stack([w1 for w1, _ in self.mlp]), dtype=like.dtype,
                                                       device=like.device)
        return hit

    def _mixer(self, layer: int) -> ChannelMix:
        key = ("mixer", layer)
        hit = self._weights.get(key)
        if hit is None:
            hit = self._weights[key] = ChannelMix(self.blocks, self.channels, self.mix[layer])
        return hit

    def energy_and_forces(self, positions, node_features, sender, receiver, shift, convolve=None):
        positions = positions.detach().requires_grad_(True)
        e = self.energy(positions, node_features, sender, receiver, shift, convolve)
        (grad,) = torch.autograd.grad(e, positions)
        return e.detach(), -grad


@dataclasses.dataclass
class EnergyWorkload:
    name: str
    model: EnergyModel
    positions: torch.Tensor      # (N, 3) float64
    node_features: torch.Tensor  # (N, X, K)
    sender: torch.Tensor
    receiver: torch.Tensor
    shift: torch.Tensor          # (E, 3) lattice translation of each edge (minimum image)

    @property
    def num_edges(self) -> int:
        return int(self.sender.shape[0])

    def to(self, device, dtype=torch.float32) -> "EnergyWorkload":
        cast = {f: getattr(self, f).to(device=device, dtype=dtype)
                for f in ("positions", "node_features", "shift")}
        return dataclasses.replace(self, sender=self.sender.to(device), receiver=self.receiver.to(device),
                                   **cast)


def config5(scale: float = 1.0) -> EnergyWorkload:
    """6 000 atoms in a periodic box (~200k edges): energy and forces through two convolutions."""
    n = max(16, int(6000 * scale))
    box = periodic_box_length(n, 30.0, 5.0)
    if box <= 10.0:
        raise ValueError("the periodic box must be wider than two cutoffs")
    pos = np.random.default_rng(41).uniform(0.0, box, size=(n, 3))
    sender, receiver, vec = radius_graph(pos, 5.0, box)
    shift = vec - (pos[sender] - pos[receiver])
    model = EnergyModel()
    x = np.random.default_rng(42).standard_normal((n, model.num_x, model.channels))
    return EnergyWorkload("cfg5", model, torch.from_numpy(pos), torch.from_numpy(x),
                          torch.from_numpy(sender), torch.from_numpy(receiver), torch.from_numpy(shift))
