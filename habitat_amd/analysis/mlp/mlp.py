"""Per-operation run-time MLPs and `RuntimePredictor`, evaluated on the GPU.

Host-side mirror of analyzer/habitat/analysis/mlp/mlp.py:17-146,252-267 for
inference: the four network classes keep the reference's layer names, so a
reference checkpoint ({'mu', 'sigma', 'model': state_dict}) loads unchanged,
and `RuntimePredictor.predict(kernel_arguments, device_name)` keeps its
signature.  The forward pass itself runs in libhabitat_mi.so
(hbt_mlp_forward: one fused fp32-MFMA kernel for the whole network);
`predict_batch` is the entry that makes it worthwhile.  Training is not part of
this package.
"""
import collections
import ctypes
import threading

import numpy as np
import torch
import torch.nn as nn
import torch.nn.functional as F

from habitat_amd import _lib
from habitat_amd.analysis.mlp.devices import get_device_features


class MLPBase(nn.Module):
    """`layers` x (Linear(layer_size, layer_size), ReLU) — mlp.py:17-31."""

    def __init__(self, layers, layer_size):
        super().__init__()
        self.layers = nn.ModuleList()
        for _ in range(layers):
            self.layers.append(nn.Linear(layer_size, layer_size))
            self.layers.append(nn.ReLU())

    def forward(self, x):
        for layer in self.layers:
            x = layer(x)
        return x


class _OperationMLP(nn.Module):
    """fc1 (features + 4 device features -> layer_size), ReLU, MLPBase, fc2 -> 1.
    The torch forward is kept for reference use on the host; prediction goes
    through the HIP library."""

    features = []

    def __init__(self, layers, layer_size):
        super().__init__()
        self.features = list(type(self).features)
        self.fc1 = nn.Linear(len(self.features) + 4, layer_size)
        self.mlp = MLPBase(layers, layer_size)
        self.fc2 = nn.Linear(layer_size, 1)

    def forward(self, x):
        return self.fc2(self.mlp(F.relu(self.fc1(x))))


class LinearMLP(_OperationMLP):       # mlp.py:34-50
    features = ["bias", "batch", "in_features", "out_features"]


class LSTMMLP(_OperationMLP):         # mlp.py:53-69
    features = ["bias", "bidirectional", "batch", "seq_len", "input_size", "hidden_size",
                "num_layers"]


class Conv2DMLP(_OperationMLP):       # mlp.py:72-90
    features = ["bias", "batch", "image_size", "in_channels", "out_channels", "kernel_size",
                "stride", "padding"]


class BMMMLP(_OperationMLP):          # mlp.py:93-109
    features = ["batch", "left", "middle", "right"]


_MODELS = {"linear": LinearMLP, "lstm": LSTMMLP, "conv2d": Conv2DMLP, "bmm": BMMMLP}


class _DeviceMLP:
    """Owner of one `hbt_mlp` handle (weights packed in HBM)."""

    def __init__(self, model, mu, sigma):
        sd = {k: v.detach().to("cpu", torch.float32).contiguous()
              for k, v in model.state_dict().items()}
        hidden = sorted(int(k.split(".")[2]) for k in sd if k.startswith("mlp.layers.")
                        and k.endswith(".weight"))
        names = ["fc1"] + ["mlp.layers.%d" % i for i in hidden] + ["fc2"]
        self._keep = [sd[n + ".weight"] for n in names] + [sd[n + ".bias"] for n in names]
        nl = len(names)
        W = (ctypes.c_void_p * nl)(*[t.data_ptr() for t in self._keep[:nl]])
        B = (ctypes.c_void_p * nl)(*[t.data_ptr() for t in self._keep[nl:]])
        mu = np.ascontiguousarray(mu, np.float64)
        sigma = np.ascontiguousarray(sigma, np.float64)
        self.in_features = int(sd["fc1.weight"].shape[1])
        width = int(sd["fc1.weight"].shape[0])
        if mu.shape != (self.in_features,) or sigma.shape != (self.in_features,):
            raise ValueError("mu/sigma must have %d entries" % self.in_features)
        err = ctypes.c_int(0)
        self.torch_device = torch.device("cuda", torch.cuda.current_device())
        self.handle = _lib.lib().hbt_mlp_create(
            self.in_features, width, len(hidden), W, B,
            mu.ctypes.data_as(ctypes.c_void_p), sigma.ctypes.data_as(ctypes.c_void_p),
            ctypes.byref(err))
        if not self.handle:
            raise _lib.HabitatLibraryError(err.value, "hbt_mlp_create")
        # Batches of up to 7168 rows (and what a larger batch leaves over) run
        # through scratch memory of the handle, so calls on one handle must not
        # overlap.  Calls that follow each other on one stream never do; a call
        # on ANOTHER stream than the one before is made to wait for that stream
        # first, under a lock that also keeps two threads apart.
        self._lock = threading.Lock()
        self._last_stream = None
        self._predict_one = _lib.lib().hbt_mlp_predict_one
        self._one_out = ctypes.c_float(0.0)       # used under self._lock
        self._one_out_ref = ctypes.byref(self._one_out)

    def _ordered_after_the_call_before(self, stream):
        """Call with self._lock held."""
        last = self._last_stream
        if last is not None and last != stream:
            stream.wait_stream(last)
        self._last_stream = stream

    def forward(self, raw, out=None, stream=None):
        """raw: [n, in_features] float64 GPU tensor -> [n] float32 GPU tensor."""
        if raw.dtype != torch.float64 or raw.dim() != 2 or raw.shape[1] != self.in_features:
            raise TypeError("raw features must be [n, %d] float64" % self.in_features)
        if raw.device != self.torch_device:
            raise ValueError("raw features must live on %s" % self.torch_device)
        raw = raw.contiguous()
        n = raw.shape[0]
        if out is None:
            out = torch.empty((n,), dtype=torch.float32, device=raw.device)
        if stream is None:
            stream = torch.cuda.current_stream(raw.device)
        with self._lock, torch.cuda.device(raw.device):
            self._ordered_after_the_call_before(stream)
            rc = _lib.lib().hbt_mlp_forward(self.handle, ctypes.c_void_p(raw.data_ptr()), n,
                                            ctypes.c_void_p(out.data_ptr()),
                                            ctypes.c_void_p(stream.cuda_stream))
        _lib.check(rc, "hbt_mlp_forward")
        return out

    def predict_one(self, row):
        """row: [in_features] float64 numpy array (host) -> float; one
        hbt_mlp_predict_one call, which waits for the result."""
        if row.dtype != np.float64 or row.shape != (self.in_features,):
            raise TypeError("one row of %d float64 features" % self.in_features)
        out = self._one_out
        index = self.torch_device.index
        with self._lock:
            # (entering torch.cuda.device costs microseconds: only when needed)
            if torch.cuda.current_device() == index:
                stream = torch.cuda.current_stream()
                self._ordered_after_the_call_before(stream)
                rc = self._predict_one(self.handle, row.ctypes.data, self._one_out_ref,
                                       stream.cuda_stream)
            else:
                with torch.cuda.device(index):
                    stream = torch.cuda.current_stream()
                    self._ordered_after_the_call_before(stream)
                    rc = self._predict_one(self.handle, row.ctypes.data, self._one_out_ref,
                                           stream.cuda_stream)
            value = out.value
        if rc != _lib.HBT_OK:
            _lib.check(rc, "hbt_mlp_predict_one")
        return value

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                _lib.lib().hbt_mlp_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


class RuntimePredictor:
    # predictions `predict` remembers: the reference asks for every operation
    # twice, once with the origin's device features (predictor.py:177-180), and
    # a trace predicted for one destination after another asks the origin-side
    # question again each time
    PREDICT_CACHE_ENTRIES = 4096

    def __init__(self, model_name, layers, layer_size, model_path=None):
        self.model_name = model_name
        self.layers = layers
        self.layer_size = layer_size
        self.model = _MODELS[self.model_name](layers, layer_size)
        self.device_params = ["mem", "mem_bw", "num_sm", "single"]
        self.mu = None
        self.sigma = None
        self._gpu = None
        self._predicted = collections.OrderedDict()
        if model_path is not None:
            self.load_state(model_path)

    # -- checkpoint format of mlp.py:133-146 ---------------------------------
    def load_state(self, path):
        # mu and sigma are numpy arrays in a reference checkpoint; allow exactly
        # those types rather than unpickling arbitrary objects.
        import numpy.core.multiarray as _ma
        allowed = [_ma._reconstruct, np.ndarray, np.dtype, type(np.dtype(np.float64)),
                   type(np.dtype(np.float32))]
        with torch.serialization.safe_globals(allowed):
            checkpoint = torch.load(path, map_location="cpu", weights_only=True)
        self.mu = np.asarray(checkpoint["mu"], np.float64)
        self.sigma = np.asarray(checkpoint["sigma"], np.float64)
        self.model.load_state_dict(checkpoint["model"])
        self.refresh()

    def save_state(self, path):
        torch.save({"mu": self.mu, "sigma": self.sigma, "model": self.model.state_dict()}, path)

    def set_normalization(self, mu, sigma):
        self.mu = np.asarray(mu, np.float64)
        self.sigma = np.asarray(sigma, np.float64)
        self.refresh()

    def refresh(self):
        """Re-upload the weights after `self.model` was modified in place (and
        forget what `predict` remembered of the old ones)."""
        self._gpu = None
        self._predicted.clear()

    def _device_mlp(self):
        if self._gpu is None:
            if self.mu is None or self.sigma is None:
                raise TypeError("mu/sigma are not set (load a checkpoint or call "
                                "set_normalization)")
            self._gpu = _DeviceMLP(self.model, self.mu, self.sigma)
        return self._gpu

    # -- prediction -----------------------------------------------------------
    def predict(self, kernel_arguments, device_name):
        """One prediction, as the reference's predict (mlp.py:252-267): one C
        call that waits for the GPU.  Asking again for the same arguments on
        the same device is answered from a table (cleared by `refresh`)."""
        device_features = get_device_features(device_name, self.device_params)
        row = list(kernel_arguments) + device_features
        features = np.array(row, dtype=np.float64)
        key = features.tobytes()
        remembered = self._predicted
        value = remembered.get(key)
        if value is not None:
            try:
                remembered.move_to_end(key)
            except KeyError:          # another thread has just dropped it
                pass
            return value
        value = self._device_mlp().predict_one(features)
        remembered[key] = value
        while len(remembered) > self.PREDICT_CACHE_ENTRIES:
            try:
                remembered.popitem(last=False)
            except KeyError:          # another thread emptied it
                break
        return value

    def predict_batch(self, raw_features, out=None, stream=None):
        """raw_features: [n, F+4] float64 (numpy array or GPU tensor): operation
        features in `self.model.features` order followed by the four device
        features.  Returns a float32 GPU tensor of n predictions (not synchronised)."""
        gpu = self._device_mlp()
        if isinstance(raw_features, np.ndarray):
            raw_features = torch.from_numpy(np.ascontiguousarray(raw_features, np.float64)).to(
                gpu.torch_device)
        return gpu.forward(raw_features, out=out, stream=stream)
