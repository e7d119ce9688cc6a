"""The reference's on-disk layout of a quantised model, for any module tree that holds LinearFLH layers.

flh/quantized_model/modeling_llama.py:1079-1137 writes it and :1139-1260 reads it: a directory with
`model.pt` -- the state dict on the CPU, float32 tensors stored as float16 (buffers `w_packed`, `w_scale`,
`w_zero`, `bias` of every quantised linear under the module's own names) -- and `quantization_config.json`
with the keys below.  The reference's model class also writes its transformers config there; that belongs
to the model code, not to this layer.
"""
import collections
import json
import os
import pickle
import zipfile

import torch

from .linear import LinearFLH

QUANT_CONFIG_DEFAULTS = {"weight_bits": 4, "weight_group_size": 128, "act_bits": 4, "act_group_size": 128,
                         "weight_sym": True, "act_sym": True, "clip_ratio": 1.0, "dtype": "float16"}


def save_quantized(module, save_directory, **quant_config):
    """Write `module`'s state dict and the quantisation settings in the reference's layout.  Keyword
    arguments override QUANT_CONFIG_DEFAULTS (unknown keys are rejected)."""
    unknown = set(quant_config) - set(QUANT_CONFIG_DEFAULTS)
    if unknown:
        raise ValueError(f"unknown quantisation settings: {sorted(unknown)}")
    os.makedirs(save_directory, exist_ok=True)
    state = {}
    for key, value in module.state_dict().items():
        value = value.detach().cpu()
        state[key] = value.half() if value.dtype == torch.float32 else value
    torch.save(state, os.path.join(save_directory, "model.pt"), pickle_protocol=4)   # as the reference writes it
    with open(os.path.join(save_directory, "quantization_config.json"), "w") as f:
        json.dump({**QUANT_CONFIG_DEFAULTS, **quant_config}, f, indent=2)


_STORAGE_DTYPES = {"HalfStorage": torch.float16, "FloatStorage": torch.float32, "DoubleStorage": torch.float64,
                   "BFloat16Storage": torch.bfloat16, "ByteStorage": torch.uint8, "CharStorage": torch.int8,
                   "ShortStorage": torch.int16, "IntStorage": torch.int32, "LongStorage": torch.int64,
                   "BoolStorage": torch.bool}


class _StorageType:
    """Stands for a torch.<X>Storage class named in the file: only its element type is used."""

    def __init__(self, dtype):
        self.dtype = dtype


def _rebuild_tensor(storage, storage_offset, size, stride, requires_grad=False, backward_hooks=None, metadata=None):
    """What torch._utils._rebuild_tensor_v2 does for a plain CPU tensor, on the flat tensor `_StateDictReader` made of
    the storage: a strided view, bounds-checked by torch."""
    return torch.as_strided(storage, tuple(size), tuple(stride), storage_offset)


class _StateDictReader(pickle.Unpickler):
    """Reads the `data.pkl` of a torch.save zip archive that holds a state dict (any pickle protocol), with an
    allow-list instead of torch's loader: the only globals that resolve are OrderedDict, the tensor rebuild function
    (replaced by the local one above) and the storage type names; anything else in the file raises.  Storages are
    read from the archive's own records."""

    def __init__(self, file, archive, prefix):
        super().__init__(file)
        self._archive, self._prefix, self._storages = archive, prefix, {}

    def find_class(self, module, name):
        if (module, name) == ("collections", "OrderedDict"):
            return collections.OrderedDict
        if (module, name) == ("torch._utils", "_rebuild_tensor_v2"):
            return _rebuild_tensor
        if module == "torch" and name in _STORAGE_DTYPES:
            return _StorageType(_STORAGE_DTYPES[name])
        raise pickle.UnpicklingError(f"model.pt names {module}.{name}: not part of a plain state dict, refused")

    def persistent_load(self, pid):
        if not (isinstance(pid, tuple) and len(pid) == 5 and pid[0] == "storage" and isinstance(pid[1], _StorageType)):
            raise pickle.UnpicklingError("unexpected persistent id in model.pt")
        _, kind, key, _location, numel = pid
        if key not in self._storages:
            raw = self._archive.read(f"{self._prefix}/data/{key}")
            flat = torch.frombuffer(bytearray(raw), dtype=kind.dtype) if raw else torch.empty(0, dtype=kind.dtype)
            if flat.numel() != numel:
                raise pickle.UnpicklingError(f"storage {key}: {flat.numel()} elements in the archive, {numel} announced")
            self._storages[key] = flat
        return self._storages[key]


def read_state_dict(path):
    """The state dict of a torch.save file, on the CPU.  Files in torch's default pickle protocol go through torch's
    own loader that executes nothing from the file (memory-mapped); files in another protocol -- the reference saves
    with protocol 4 (flh/quantized_model/modeling_llama.py:1107), which that loader refuses -- through the allow-list
    reader above.  Neither runs code from the file."""
    import warnings
    try:
        with warnings.catch_warnings():
            warnings.simplefilter("ignore", UserWarning)       # torch announces the other protocol before it gives up
            return torch.load(path, map_location="cpu", mmap=True, weights_only=True)
    except pickle.UnpicklingError:
        pass
    with zipfile.ZipFile(path) as archive:
        names = [n for n in archive.namelist() if n.endswith("/data.pkl")]
        if len(names) != 1:
            raise pickle.UnpicklingError(f"{path}: not a torch.save archive")
        prefix = names[0][: -len("/data.pkl")]
        with archive.open(names[0]) as f:
            state = _StateDictReader(f, archive, prefix).load()
    if not isinstance(state, dict) or not all(isinstance(k, str) and torch.is_tensor(v) for k, v in state.items()):
        raise pickle.UnpicklingError(f"{path}: not a state dict of tensors")
    return state


def load_quantized(module, load_directory, device=None, strict=True):
    """Fill `module` (already built with the right structure) from a directory written by save_quantized or by
    the reference's `save_quantized`; returns the quantisation settings.  Nothing from the file is executed
    (read_state_dict)."""
    with open(os.path.join(load_directory, "quantization_config.json")) as f:
        quant_config = {**QUANT_CONFIG_DEFAULTS, **json.load(f)}
    state = read_state_dict(os.path.join(load_directory, "model.pt"))
    group = quant_config["weight_group_size"]
    own = module.state_dict()
    for name, layer in module.named_modules():
        if not isinstance(layer, LinearFLH):
            continue
        key = f"{name}.w_scale" if name else "w_scale"
        if key in state and key in own and tuple(state[key].shape) != tuple(own[key].shape):
            raise ValueError(f"{key}: stored scales {tuple(state[key].shape)} do not fit a layer built for "
                             f"{tuple(own[key].shape)} (weight_group_size in the file: {group})")
    for key in list(state):
        if state[key].dtype == torch.float32:
            state[key] = state[key].half()
    result = module.load_state_dict(state, strict=strict)
    for layer in module.modules():
        if isinstance(layer, LinearFLH):
            layer.drop_six_bit_weights()
    if device is not None:
        module.to(device)
    quant_config["missing_keys"], quant_config["unexpected_keys"] = list(result.missing_keys), list(result.unexpected_keys)
    return quant_config
