"""GradientClipper and AdamOptimizer with the reference's surface, running as multi-tensor
device kernels.

Reference: src/RMAD/GradientClipper.cs:31-71 (Clip over layers), :118-157 (ClipGradients);
src/RMAD/AdamOptimizer.cs:32-91 (Optimize over layers), :195-239 (UpdateWeightWithAdam);
parameters and defaults from src/RMAD/NeuralNetworkParameters.cs:18-88 (PRADLite:
lite/src/ParallelReverseAutoDiffLite/Lite/NeuralNetworkParameters.cs).
"""
from . import _lib
from .exceptions import InvalidOperationException, check
from .matrix import DeepMatrix, Matrix
from .operations import _ensure_initialized, handle_array


class NeuralNetworkParameters:
    """The fields of the reference's parameter object that this path reads."""

    def __init__(self, lite=False):
        self.BatchSize = 8
        self.LeakyReLUAlpha = 0.01
        self.LearningRate = 0.001
        self.AdamIteration = 1.0
        self.AdamBeta1 = 0.9
        self.AdamBeta2 = 0.999
        self.AdamEpsilon = 1e-8
        self.ClipValue = 4.0
        self.MinimumClipValue = 1e-8 if lite else 1e-16


class ModelLayer:
    """Named (weight, gradient, first moment, second moment) groups of one layer: the part of
    src/RMAD/ModelLayer.cs / IModelLayer.cs that clip and Adam read (Identifiers, Dimensions,
    layer[identifier, ModelElementType])."""

    def __init__(self):
        self.Identifiers = []
        self._elements = {}

    def AddModelElementGroup(self, identifier, weight, gradient=None, first_moment=None, second_moment=None):
        def like(m):
            if isinstance(m, DeepMatrix):
                return DeepMatrix(m.Depth, m.Rows, m.Cols, m.dtype)
            return Matrix(m.Rows, m.Cols, m.dtype)
        self.Identifiers.append(identifier)
        self._elements[identifier] = {
            "Weight": weight,
            "Gradient": gradient if gradient is not None else like(weight),
            "FirstMoment": first_moment if first_moment is not None else like(weight),
            "SecondMoment": second_moment if second_moment is not None else like(weight),
        }
        return self

    def __getitem__(self, key):
        identifier, element = key
        return self._elements[identifier][element]

    def Dimensions(self, identifier):
        w = self._elements[identifier]["Weight"]
        if isinstance(w, DeepMatrix):
            return [w.Depth, w.Rows, w.Cols]
        return [w.Rows, w.Cols]

    def WeightMatrix(self, identifier):
        return self[identifier, "Weight"]

    def GradientMatrix(self, identifier):
        return self[identifier, "Gradient"]


class _Net:
    def __init__(self, parameters):
        self.Parameters = parameters


def _collect(layers, element):
    out = []
    for layer in layers:
        for identifier in layer.Identifiers:
            m = layer[identifier, element]
            if m is None:
                raise InvalidOperationException("%s cannot be null." % element)
            out.append(m)
    return out


class GradientClipper:
    def __init__(self, network):
        self.network = network if hasattr(network, "Parameters") else _Net(network)

    def Clip(self, layers):
        """Standardise-and-clamp every gradient of every layer in place (one launch sequence)."""
        _ensure_initialized()
        grads = _collect(layers, "Gradient")
        if not grads:
            return
        p = self.network.Parameters
        bufs = [g.device() for g in grads]
        for dtype in {b.dtype for b in bufs}:
            group = [b for b in bufs if b.dtype == dtype]
            check(_lib.load().prad_clip_multi(handle_array(group), len(group), float(p.ClipValue), float(p.MinimumClipValue)))
        for g in grads:
            _mark_written(g)


class AdamOptimizer:
    def __init__(self, network):
        self.network = network if hasattr(network, "Parameters") else _Net(network)

    def Optimize(self, layers):
        """One Adam step on every (w, m, v, g) group of every layer, in place on the device."""
        _ensure_initialized()
        w = _collect(layers, "Weight")
        if not w:
            return
        m = _collect(layers, "FirstMoment")
        v = _collect(layers, "SecondMoment")
        g = _collect(layers, "Gradient")
        p = self.network.Parameters
        wb, mb, vb, gb = ([x.device() for x in xs] for xs in (w, m, v, g))
        for dtype in {b.dtype for b in wb}:
            idx = [i for i, b in enumerate(wb) if b.dtype == dtype]
            check(_lib.load().prad_adam_multi(
                handle_array([wb[i] for i in idx]), handle_array([mb[i] for i in idx]),
                handle_array([vb[i] for i in idx]), handle_array([gb[i] for i in idx]), len(idx),
                float(p.LearningRate), float(p.AdamBeta1), float(p.AdamBeta2), float(p.AdamEpsilon), float(p.AdamIteration)))
        for x in w + m + v:
            _mark_written(x)


def _mark_written(m):
    if isinstance(m, DeepMatrix):
        for s in m:
            s._device_written()
    else:
        m._device_written()
