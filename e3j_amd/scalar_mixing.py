"""Index map of the per-irrep scalar mixing (`src/e3j/core/scalar_mixing.py:57-67`).

`out[.., i, c] = s[.., mix_indices[i], c] * x[.., i, c]`: every irreducible
block of the feature space (one per Clebsch-Gordan path, counted with
multiplicity) is scaled by its own scalar.  The product itself is evaluated
inside the fused convolution kernels; only the index map lives on the host.
"""

from __future__ import annotations

import numpy as np

from .options import Layout
from .spaces import O3Space


class ScalarMixing:
    def __init__(self, source, layout=Layout.TRAILING_CHANNELS):
        self.source = O3Space(source)
        self.layout = Layout.parse(layout)

    @property
    def num_irreps(self) -> int:
        return self.source.num_irreps

    @property
    def mix_indices(self) -> np.ndarray:
        repeats = []
        for mul, ir in self.source:
            repeats.extend([ir.dim] * mul)
        return np.repeat(np.arange(self.num_irreps), repeats)
