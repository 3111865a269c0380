"""Lifecycle shared by perturbed layers: the part of the reference's ``modules/base.py`` that the binary
layers inherit (``Perturbed`` modules/base.py:44-108, ``PerturbedModel`` modules/base.py:9-41).  The float
NES layers of that file (Perturbed*/Permuted*/Synthetic* Linear/Conv2d) run on stock torch ops and are not
part of this package."""
import random

import torch  # noqa: F401  (kept so `from modules.base import *` exposes torch like the reference)
from torch import nn  # noqa: F401


class Perturbed:
    """Mixin holding the per-population noise state of one layer.

    Attributes (same names as the reference): ``directions`` (population size), ``perturbed_flag``
    (set by :class:`PerturbedModel` around a forward), ``noise_scale``, ``seed``, ``antithetic``,
    ``options``, ``weight_noise`` / ``bias_noise`` (per-member tensors or ``None``)."""

    def __init__(self, directions, antithetic=False, options=None):
        self.directions = directions
        self.perturbed_flag = False
        self.noise_scale = None
        self.seed = None
        self.antithetic = antithetic
        self.options = {} if options is None else options
        # The reference calls free_memory() here, which reads self.bias before the binary layers have
        # assigned it (modules/base.py:54,107 vs modules/binary.py:86-88); set the fields directly.
        self.weight_noise = None
        self.bias_noise = None

    def set_noise_scale(self, noise_scale):
        self.noise_scale = noise_scale

    def set_noise(self, noise_scale=None):
        """Draw this layer's per-member noise; provided by the concrete layer."""
        raise NotImplementedError

    def update(self, weights, l1=0, l2=0):
        """Turn per-member fitness weights into gradients; provided by the concrete layer."""
        raise NotImplementedError

    def set_seed(self, seed=None):
        """modules/base.py:88-89."""
        self.seed = seed if seed is not None else random.randrange(100000000)

    def allocate_weight(self):
        self.weight_noise = torch.empty((self.directions,) + tuple(self.weight.size()),
                                        device=self.weight.device, dtype=self.weight.dtype)

    def allocate_bias(self):
        if getattr(self, "bias", None) is not None:
            self.bias_noise = torch.empty((self.directions,) + tuple(self.bias.size()),
                                          device=self.bias.device, dtype=self.bias.dtype)

    def allocate_memory(self):
        self.allocate_weight()
        self.allocate_bias()

    def free_memory(self):
        """Drop the per-member tensors (called before pickling a model, README.md:107)."""
        self.weight_noise = None
        self.bias_noise = None


class PerturbedModel:
    """Wraps a model, finds its :class:`Perturbed` layers and fans lifecycle calls out to them
    (modules/base.py:9-41): ``forward`` raises ``perturbed_flag`` on every layer for the duration of the
    call; any other attribute is a method broadcast to the layers when ``Perturbed`` defines it
    (``set_noise``, ``set_seed``, ``update``, ``free_memory`` ...) and otherwise a call on the wrapped model
    made with the flags raised."""

    def __init__(self, model, directions):
        self.model = model
        self.directions = directions
        self.perturbed_layers = []

        def collect(m):
            if isinstance(m, Perturbed):
                self.perturbed_layers.append(m)

        self.model.apply(collect)

    def _flags(self, value):
        for layer in self.perturbed_layers:
            layer.perturbed_flag = value

    def forward(self, input, *args):
        self._flags(True)
        try:
            return self.model.forward(input, *args)
        finally:
            self._flags(False)

    def __getattr__(self, name):
        def fan_out(*args, **kwargs):
            if hasattr(Perturbed, name):
                for layer in self.perturbed_layers:
                    getattr(layer, name)(*args, **kwargs)
                return None
            self._flags(True)
            try:
                return getattr(self.model, name)(*args, **kwargs)
            finally:
                self._flags(False)

        return fan_out
