"""MLX-format safetensors ingestion for the quantized-matmul path.

Host-side mirror of the reference loader (crates/rmlx-nn/src/safetensors_loader.rs): the
`quantization` block of `config.json` (:126-162), the `.weight` / `.scales` / `.biases` triplet
detection (:420-478) and `assemble_quantized_linear` (:495-552).  The MLX uint32 word layout is the
layout the kernels consume, so the reference's `repack_mlx_weight` to bytes (:562-628) is the
identity on the little-endian byte view and no repacking happens here; weights, scales and biases
are uploaded once and stay on the device (the reference re-uploads them on every forward,
crates/rmlx-nn/src/quantized_linear.rs:189).

The safetensors container is parsed here directly (8-byte little-endian header length, JSON header
with dtype / shape / data_offsets per tensor, raw little-endian data): nothing from the file is
executed and no third-party reader is needed.
"""
import json
import os
import struct

import numpy as np

from . import ops
from .runtime import DeviceBuffer, F16, F32, U32, U8, BF16


class SafetensorsLoadError(Exception):
    """Mirror of `SafetensorsLoadError` (safetensors_loader.rs:37-78): `kind` is one of
    Io, Parse, TensorNotFound, UnsupportedDtype, InvalidQuantConfig, QuantizedLinearError."""

    def __init__(self, kind, message):
        super().__init__(f"{kind}: {message}")
        self.kind = kind


class QuantizationConfig:
    """`QuantizationConfig` (safetensors_loader.rs:100-110)."""

    def __init__(self, bits, group_size):
        self.bits, self.group_size = int(bits), int(group_size)

    def __eq__(self, other):
        return (self.bits, self.group_size) == (other.bits, other.group_size)

    def __repr__(self):
        return f"QuantizationConfig(bits={self.bits}, group_size={self.group_size})"


def parse_quantization_config(path):
    """`parse_quantization_config` (safetensors_loader.rs:126-162): None when config.json has no
    `quantization` block; bits must be 4 or 8 and group_size 32, 64 or 128."""
    try:
        with open(path, "r", encoding="utf-8") as f:
            content = f.read()
    except OSError as e:
        raise SafetensorsLoadError("Io", str(e))
    try:
        cfg = json.loads(content)
    except ValueError as e:
        raise SafetensorsLoadError("Parse", str(e))
    quant = cfg.get("quantization") if isinstance(cfg, dict) else None
    if quant is None:
        return None
    bits, group_size = quant.get("bits"), quant.get("group_size")
    if not isinstance(bits, int) or isinstance(bits, bool) or bits < 0:
        raise SafetensorsLoadError("InvalidQuantConfig", "missing or invalid 'bits' field")
    if not isinstance(group_size, int) or isinstance(group_size, bool) or group_size < 0:
        raise SafetensorsLoadError("InvalidQuantConfig", "missing or invalid 'group_size' field")
    if bits not in (4, 8):
        raise SafetensorsLoadError("InvalidQuantConfig", f"bits must be 4 or 8, got {bits}")
    if group_size not in (32, 64, 128):
        raise SafetensorsLoadError("InvalidQuantConfig", f"group_size must be 32, 64, or 128, got {group_size}")
    return QuantizationConfig(bits, group_size)


def hf_name_to_rmlx(hf_name):
    """`hf_name_to_rmlx` (safetensors_loader.rs:234-248)."""
    name = hf_name[len("model."):] if hf_name.startswith("model.") else hf_name
    for old, new in (("self_attn.", "attention."), ("mlp.gate_proj.", "feed_forward.gate_proj."),
                     ("mlp.up_proj.", "feed_forward.up_proj."), ("mlp.down_proj.", "feed_forward.down_proj."),
                     ("input_layernorm.", "attention_norm."), ("post_attention_layernorm.", "ffn_norm."),
                     ("embed_tokens.", "embedding."), ("model.norm.", "norm.")):
        name = name.replace(old, new)
    return name


# safetensors dtype -> (numpy dtype of the raw data, device dtype tag); the reference maps the same
# set (safetensors_loader.rs:168-182) and rejects the rest.
_DTYPES = {"F32": (np.dtype("<f4"), F32), "F16": (np.dtype("<f2"), F16), "BF16": (np.dtype("<u2"), BF16),
           "U32": (np.dtype("<u4"), U32), "U8": (np.dtype("u1"), U8)}


class SafetensorsFile:
    """Parsed container: tensor name -> (dtype string, shape, numpy view of the raw data)."""

    def __init__(self, path):
        try:
            size = os.path.getsize(path)
            with open(path, "rb") as f:
                head = f.read(8)
                if len(head) != 8:
                    raise SafetensorsLoadError("Parse", "file shorter than the 8-byte header length")
                (hlen,) = struct.unpack("<Q", head)
                if hlen > size - 8 or hlen > (100 << 20):
                    raise SafetensorsLoadError("Parse", f"invalid header length {hlen}")
                header_bytes = f.read(hlen)
        except OSError as e:
            raise SafetensorsLoadError("Io", str(e))
        try:
            header = json.loads(header_bytes.decode("utf-8"))
        except ValueError as e:
            raise SafetensorsLoadError("Parse", str(e))
        if not isinstance(header, dict):
            raise SafetensorsLoadError("Parse", "header is not a JSON object")
        self.metadata = header.pop("__metadata__", None)
        self._data = np.memmap(path, dtype=np.uint8, mode="r", offset=8 + hlen) if size > 8 + hlen else np.zeros(0, np.uint8)
        self.entries = {}
        for name, info in header.items():
            try:
                dtype, shape, (lo, hi) = info["dtype"], [int(s) for s in info["shape"]], info["data_offsets"]
            except (KeyError, TypeError, ValueError) as e:
                raise SafetensorsLoadError("Parse", f"tensor {name}: bad header entry ({e})")
            if not (0 <= lo <= hi <= self._data.size):
                raise SafetensorsLoadError("Parse", f"tensor {name}: data_offsets {lo}..{hi} outside the file")
            self.entries[name] = (dtype, shape, lo, hi)

    def names(self):
        return list(self.entries.keys())

    def tensor(self, name):
        """(dtype string, shape, numpy array over the mapped bytes)."""
        if name not in self.entries:
            raise SafetensorsLoadError("TensorNotFound", name)
        dtype, shape, lo, hi = self.entries[name]
        if dtype not in _DTYPES:
            raise SafetensorsLoadError("UnsupportedDtype", f"tensor {name}: {dtype}")
        np_dtype = _DTYPES[dtype][0]
        count = int(np.prod(shape, dtype=np.int64)) if shape else 1
        if (hi - lo) != count * np_dtype.itemsize:
            raise SafetensorsLoadError("Parse", f"tensor {name}: {hi - lo} bytes for shape {shape} of {dtype}")
        return dtype, shape, np.frombuffer(self._data[lo:hi], dtype=np_dtype).reshape(shape)


class SafetensorsWeightMap:
    """`SafetensorsWeightMap` (safetensors_loader.rs:255-337): plain tensors by name and quantized
    linear layers by prefix, both resident on the device."""

    def __init__(self, tensors=None, quantized_layers=None):
        self.tensors = tensors or {}
        self.quantized_layers = quantized_layers or {}

    def __len__(self):
        return len(self.tensors)

    def is_empty(self):
        return not self.tensors

    def get(self, name):
        if name not in self.tensors:
            raise SafetensorsLoadError("TensorNotFound", name)
        return self.tensors[name]

    def take(self, name):
        if name not in self.tensors:
            raise SafetensorsLoadError("TensorNotFound", name)
        return self.tensors.pop(name)

    def contains(self, name):
        return name in self.tensors

    def names(self):
        return list(self.tensors.keys())

    def get_quantized(self, prefix):
        return self.quantized_layers.get(prefix)

    def take_quantized(self, prefix):
        return self.quantized_layers.pop(prefix, None)

    def num_quantized(self):
        return len(self.quantized_layers)

    def quantized_names(self):
        return list(self.quantized_layers.keys())


def find_triplets(names):
    """prefix -> (weight, scales, biases) for every `.weight` that has both companions
    (safetensors_loader.rs:432-447)."""
    have = set(names)
    out = {}
    for name in names:
        if name.endswith(".weight"):
            prefix = name[:-len(".weight")]
            if f"{prefix}.scales" in have and f"{prefix}.biases" in have:
                out[prefix] = (name, f"{prefix}.scales", f"{prefix}.biases")
    return out


def _upload(dtype, array):
    return DeviceBuffer.from_numpy(np.ascontiguousarray(array), _DTYPES[dtype][1])


def assemble_quantized_linear(st, prefix, names, qc):
    """`assemble_quantized_linear` (safetensors_loader.rs:495-552): weight u32 [out, in/pack],
    scales / biases f16 [out, in/group_size]."""
    w_dtype, w_shape, w = st.tensor(names[0])
    s_dtype, s_shape, s = st.tensor(names[1])
    b_dtype, b_shape, b = st.tensor(names[2])
    if len(w_shape) != 2 or len(s_shape) != 2:
        raise SafetensorsLoadError("InvalidQuantConfig",
                                   f"{prefix}: weight shape {w_shape} or scales shape {s_shape} is not 2D")
    if qc.bits not in (4, 8):
        raise SafetensorsLoadError("InvalidQuantConfig", f"unsupported bits: {qc.bits}")
    if w_dtype != "U32" or s_dtype != "F16" or b_dtype != "F16":
        raise SafetensorsLoadError("QuantizedLinearError",
                                   f"{prefix}: expected U32 weight and F16 scales/biases, got {w_dtype}/{s_dtype}/{b_dtype}")
    out_features, in_features = w_shape[0], w_shape[1] * (32 // qc.bits)
    try:  # validation (and its messages) is QuantizedLinear::new's (quantized_linear.rs:77-150)
        return ops.QuantizedLinear(w.reshape(-1).view(np.uint8), s.astype(np.float32), b.astype(np.float32),
                                   in_features, out_features, qc.group_size, qc.bits)
    except ops.KernelError as e:
        raise SafetensorsLoadError("QuantizedLinearError", f"{prefix}: {e}")


def load_safetensors_weights(path, quant_config=None):
    """`load_safetensors_weights` (safetensors_loader.rs:347-362)."""
    st = SafetensorsFile(path)
    names = st.names()
    triplets = find_triplets(names) if quant_config is not None else {}
    members = {n for t in triplets.values() for n in t}
    tensors, quantized = {}, {}
    for name in names:
        if name in members:
            continue
        dtype, _, array = st.tensor(name)
        tensors[name] = _upload(dtype, array)
    for prefix, t in triplets.items():
        quantized[prefix] = assemble_quantized_linear(st, prefix, t, quant_config)
    return SafetensorsWeightMap(tensors, quantized)


def load_safetensors_sharded(paths, quant_config=None):
    """`load_safetensors_sharded` (safetensors_loader.rs:367-385): later shards override."""
    out = SafetensorsWeightMap()
    for path in paths:
        part = load_safetensors_weights(path, quant_config)
        out.tensors.update(part.tensors)
        out.quantized_layers.update(part.quantized_layers)
    return out


def write_safetensors(path, tensors):
    """Writes `{name: (dtype string, numpy array)}` in safetensors layout (used by the tests to
    build MLX-style checkpoints; data 8-byte aligned like the reference writers)."""
    header, blobs, offset = {}, [], 0
    for name, (dtype, array) in tensors.items():
        raw = np.ascontiguousarray(array, _DTYPES[dtype][0]).tobytes()
        header[name] = {"dtype": dtype, "shape": list(np.shape(array)), "data_offsets": [offset, offset + len(raw)]}
        blobs.append(raw)
        offset += len(raw)
    hbytes = json.dumps(header, separators=(",", ":")).encode("utf-8")
    hbytes += b" " * ((8 - len(hbytes) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hbytes)))
        f.write(hbytes)
        for raw in blobs:
            f.write(raw)
