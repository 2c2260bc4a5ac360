"""End-to-end energy and forces through two stacked convolutions (the 64-channel lmax-3
configuration): gradients with respect to the atom positions flow through the spherical
harmonics and the radial network into the fused kernels' VJPs."""

import numpy as np
import pytest
import torch

from e3j_amd import workloads as W
from tests import helpers as H

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def reference():
    w = W.config5(0.02)
    host = w.to("cpu", torch.float64)
    energy, forces = w.model.energy_and_forces(host.positions, host.node_features, host.sender,
                                               host.receiver, host.shift, H.dense_convolve(w.model))
    return w, host, energy, forces


def test_float64_energy_and_forces_match_the_dense_form(reference):
    w, _, energy, forces = reference
    d = w.to("cuda", torch.float64)
    e, f = w.model.energy_and_forces(d.positions, d.node_features, d.sender, d.receiver, d.shift)
    torch.testing.assert_close(e.cpu(), energy, rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(f.cpu(), forces, rtol=1e-8, atol=1e-9 * float(forces.abs().max()))


def test_float32_energy_and_forces(reference):
    """fp32 through the compile-time-unrolled kernels: 1e-5 on the energy, and on the forces
    1e-4 of the largest force component (two layers of fp32 sums feed each gradient)."""
    w, _, energy, forces = reference
    d = w.to("cuda", torch.float32)
    e, f = w.model.energy_and_forces(d.positions, d.node_features, d.sender, d.receiver, d.shift)
    assert f.dtype == torch.float32 and f.shape == forces.shape
    torch.testing.assert_close(e.double().cpu(), energy, rtol=1e-5, atol=1e-5 * float(energy.abs()) + 1e-6)
    scale = float(forces.abs().max())
    assert float((f.double().cpu() - forces).abs().max()) <= 1e-4 * scale
    # Newton's third law on a periodic cell: the forces sum to zero (translation invariance)
    assert float(f.double().sum(0).abs().max()) <= 1e-4 * scale * np.sqrt(forces.shape[0])


def test_whole_step_replays_from_a_captured_graph():
    """Energy and forces (both convolutions, their VJPs, the harmonics kernels and the tensor
    glue around them) recorded once into a HIP graph and replayed on moved atoms: every replay
    agrees with the eager step on the same positions.  The adjacency is prepared before the
    capture (the operators keep it for the index tensors they have seen)."""
    w = W.config5(0.1)
    d = w.to("cuda", torch.float32)
    model = w.model
    pos = d.positions.clone()

    def step():
        return model.energy_and_forces(pos, d.node_features, d.sender, d.receiver, d.shift)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        energy, forces = step()
    moves = torch.Generator(device="cuda").manual_seed(3)
    for _ in range(3):
        pos.copy_(d.positions + 0.05 * torch.randn(pos.shape, device="cuda", generator=moves))
        graph.replay()
        torch.cuda.synchronize()
        got_e, got_f = energy.clone(), forces.clone()
        want_e, want_f = step()   # eager work between the replays
        torch.cuda.synchronize()
        torch.testing.assert_close(got_e, want_e, rtol=1e-5, atol=1e-6)
        assert float((got_f - want_f).abs().max()) <= 1e-5 * float(want_f.abs().max())
    assert float((want_f - forces).abs().max()) <= 1e-5 * float(want_f.abs().max())


def test_full_size_energy_and_forces_through_their_invariances():
    """The configuration at its full size (6 000 atoms, ~180k edges, 64 channels), through what the
    physics fixes for any size: the forces sum to zero; a rigid translation of all atoms leaves
    energy and forces unchanged; a rotation of all atoms (lattice translations of the edges and the
    node features turned with it, by the Wigner matrices of their degrees) leaves the energy
    unchanged and turns the forces; a HIP-graph replay of the whole step equals the eager step."""
    from scipy.spatial.transform import Rotation
    from tests.test_gpu_ops import _wigner_d
    w = W.config5(1.0)
    assert w.positions.shape[0] == 6000 and 150_000 < w.num_edges < 250_000
    d = w.to("cuda", torch.float32)
    model = w.model
    n = d.positions.shape[0]

    def step(pos, feats, shift):
        return model.energy_and_forces(pos, feats, d.sender, d.receiver, shift)

    e0, f0 = step(d.positions, d.node_features, d.shift)
    torch.cuda.synchronize()
    scale = float(f0.abs().max())
    assert np.isfinite(float(e0)) and scale > 0
    e_tol = 1e-5 * n                       # atoms contribute O(1) each, in float32
    # Newton's third law on the periodic cell
    assert float(f0.double().sum(0).abs().max()) <= 1e-4 * scale * np.sqrt(n)
    # rigid translation: the edge vectors are the same up to the rounding of the moved positions
    t = torch.tensor([1.7, -0.4, 2.9], device="cuda")
    e1, f1 = step(d.positions + t, d.node_features, d.shift)
    assert abs(float(e1) - float(e0)) <= e_tol
    assert float((f1 - f0).abs().max()) <= 2e-4 * scale
    # rotation: positions and lattice translations turn with R, node features with D(R)
    rot = Rotation.from_rotvec([0.5, -0.3, 0.8]).as_matrix()
    wig = torch.as_tensor(_wigner_d(model.layers[0].source[0], rot), dtype=torch.float64)
    r32 = torch.as_tensor(rot, dtype=torch.float32, device="cuda")
    feats = torch.einsum("ij,njc->nic", wig, w.node_features.double()).to("cuda", torch.float32)
    pos_r = (w.positions.double() @ torch.as_tensor(rot).T).to("cuda", torch.float32)
    shift_r = (w.shift.double() @ torch.as_tensor(rot).T).to("cuda", torch.float32)
    e2, f2 = step(pos_r, feats, shift_r)
    assert abs(float(e2) - float(e0)) <= e_tol
    assert float((f2 - f0 @ r32.T).abs().max()) <= 2e-4 * scale
    # the whole step from a captured graph, on moved atoms, with eager work between the replays
    pos = d.positions.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(pos, d.node_features, d.shift)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ge, gf = step(pos, d.node_features, d.shift)
    moves = torch.Generator(device="cuda").manual_seed(5)
    for _ in range(2):
        pos.copy_(d.positions + 0.05 * torch.randn(pos.shape, device="cuda", generator=moves))
        graph.replay()
        torch.cuda.synchronize()
        got_e, got_f = ge.clone(), gf.clone()
        want_e, want_f = step(pos, d.node_features, d.shift)
        torch.cuda.synchronize()
        assert abs(float(got_e) - float(want_e)) <= e_tol
        assert float((got_f - want_f).abs().max()) <= 1e-5 * float(want_f.abs().max())
