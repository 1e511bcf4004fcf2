"""GradientClipper and AdamOptimizer with the reference's surface, running as multi-tensor
device kernels.

Reference: src/RMAD/GradientClipper.cs:31-71 (Clip over layers), :118-157 (ClipGradients);
src/RMAD/AdamOptimizer.cs:32-91 (Optimize over layers), :195-239 (UpdateWeightWithAdam);
parameters and defaults from src/RMAD/NeuralNetworkParameters.cs:18-88 (PRADLite:
lite/src/ParallelReverseAutoDiffLite/Lite/NeuralNetworkParameters.cs).
"""
import json

import numpy as np

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

    # ---- files (src/RMAD/ModelLayer.cs:219-320): Newtonsoft JSON of the Matrix / DeepMatrix converters; the
    # (weights, firstMoments, secondMoments) tuple serializes as {"Item1": .., "Item2": .., "Item3": ..}.  Values
    # that live on the device are downloaded for saving; loaded values replace the element objects and reach
    # the device on their next use.
    def _dump(self, element):
        return {i: self._elements[i][element].to_json_object() for i in self.Identifiers}

    def _load(self, objects, element):
        for identifier, obj in objects.items():
            if identifier in self._elements:       # unknown identifiers in the file are ignored, as in the reference
                current = self._elements[identifier][element]
                kind = DeepMatrix if isinstance(current, DeepMatrix) else Matrix
                self._elements[identifier][element] = kind.from_json_object(obj, current.dtype)

    def SaveWeights(self, path):
        with open(path, "w") as f:
            json.dump(self._dump("Weight"), f, indent=2)

    def LoadWeights(self, path):
        with open(path) as f:
            weights = json.load(f)
        if weights is None:
            raise InvalidOperationException("Weights must not be null.")
        self._load(weights, "Weight")

    def SaveWeightsAndMoments(self, path):
        with open(path, "w") as f:
            json.dump({"Item1": self._dump("Weight"), "Item2": self._dump("FirstMoment"), "Item3": self._dump("SecondMoment")},
                      f, indent=2)

    def LoadWeightsAndMoments(self, path):
        with open(path) as f:
            items = json.load(f)
        self._load(items["Item1"], "Weight")
        self._load(items["Item2"], "FirstMoment")
        self._load(items["Item3"], "SecondMoment")

    # ---- HDF5 files (src/RMAD/ModelLayer.cs:258-271): <path>.json names what is stored, <path>.hdf5 holds the rows
    # of every weight, first moment and second moment.  Loading replaces the rows of the existing element objects.
    _BINARY_GETS = (lambda e: e["Weight"], lambda e: e["FirstMoment"], lambda e: e["SecondMoment"])

    def _ordered_elements(self):
        return {i: self._elements[i] for i in self.Identifiers}

    def SaveWeightsAndMomentsBinary(self, path):
        from . import hdf5
        if not hdf5.SerializeElements(path, self._ordered_elements(), self._BINARY_GETS):
            self.SaveWeightsAndMoments(str(path) + ".json")

    def LoadWeightsAndMomentsBinary(self, path):
        from . import hdf5
        hdf5.DeserializeElements(path, self._elements, self._BINARY_GETS)

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


class GradientClearer:
    """src/RMAD/GradientClearer.cs:21-86: every gradient of every layer back to zero.  The reference replaces each
    row by a new zero array; a gradient that lives on the device is zero-filled there instead (one launch, no copy),
    a host-only one gets new zero rows as in the reference."""

    def Clear(self, layers):
        on_device = []
        for g in _collect(layers, "Gradient"):
            for m in (g if isinstance(g, DeepMatrix) else [g]):
                if m._dev is not None:
                    on_device.append(m)
                else:
                    for i in range(m.Rows):
                        m[i] = np.zeros(m.Cols, dtype=m.dtype)
        if on_device:  # one launch for all of them
            check(_lib.load().prad_zero_multi(handle_array([m._dev for m in on_device]), len(on_device)))
            for m in on_device:
                m._device_written()


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
        self._apply(layers, "prad_adam_multi")

    def Revert(self, layers):
        """Undoes the last update (src/RMAD/AdamOptimizer.cs:97-156): as in the reference, the gradients must still be
        those of that update and Parameters.AdamIteration the iteration it was made with."""
        self._apply(layers, "prad_adam_revert_multi")

    def _apply(self, layers, entry_point):
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
            check(getattr(_lib.load(), entry_point)(
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
