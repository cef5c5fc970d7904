"""The reference's serde representation of a tensor (src/tensor.rs:1199-1249, :2181-2232), so that
tensors written by one side load on the other.

The reference derives `Serialize` for `struct Tensor { dim, buffer }`; `dim` is ndarray's fixed-rank
dimension (a tuple of u64) and `buffer` is krnl's `Buffer` tuple struct `(scalar type name, element
count, sequence of u64)`.  The u64 items are the buffer's bytes taken eight at a time, each group
read as a BIG-endian integer (the token test at src/tensor.rs:2236-2277 pins this: the u32 values
1, 2 give the item 0x0100000002000000).  krnl is not part of the reference tree: how a byte count
that is not a multiple of eight ends is not pinned by anything there; this module pads the last
group with zero bytes (parity unpinned for that case).

Two encodings are provided: the token stream of the reference's own test, and what `serde_json`
makes of the same data model (`{"dim":[..],"buffer":["F32",n,[..]]}`), the one self-describing
format in the reference's dependency list (Cargo.toml:25).

The data travel in standard layout: the reference serialises the buffer it holds, which for a
contiguous tensor is exactly that; a view that is not contiguous is copied first here.
"""
import json

import numpy as np

# krnl's ScalarType variant names for the element types a host array can carry here
_NAME_OF = {"uint8": "U8", "int8": "I8", "uint16": "U16", "int16": "I16", "uint32": "U32", "int32": "I32",
            "float32": "F32", "uint64": "U64", "int64": "I64", "float64": "F64", "float16": "F16"}
_DTYPE_OF = {v: np.dtype(k) for k, v in _NAME_OF.items()}
_DTYPE_OF["BF16"] = np.dtype("uint16")  # bf16 travels as its bit patterns


class SerdeError(ValueError):
    pass


def _items(array):
    raw = np.ascontiguousarray(array).tobytes()  # little-endian memory image, as on the reference's hosts
    raw += b"\0" * (-len(raw) % 8)
    return [int(v) for v in np.frombuffer(raw, dtype=">u8")]


def _from_items(items, name, count):
    if name not in _DTYPE_OF:
        raise SerdeError(f"unknown scalar type {name!r}")
    dt = _DTYPE_OF[name]
    need = -(-count * dt.itemsize // 8)
    if len(items) != need:
        raise SerdeError(f"buffer of {count} {name} needs {need} items, found {len(items)}")
    for v in items:
        if not isinstance(v, int) or isinstance(v, bool) or v < 0 or v >= 1 << 64:
            raise SerdeError(f"buffer item {v!r} is not a u64")
    raw = np.array(items, dtype=">u8").tobytes()[:count * dt.itemsize]
    return np.frombuffer(raw, dtype=dt).copy()


def scalar_name(array, bf16=False):
    if bf16:
        if array.dtype != np.uint16:
            raise SerdeError("bf16 data are uint16 bit patterns")
        return "BF16"
    try:
        return _NAME_OF[array.dtype.name]
    except KeyError:
        raise SerdeError(f"no scalar type for dtype {array.dtype}") from None


def to_tokens(array, bf16=False):
    """The serde_test token stream of the reference's `tensor_serde` test (src/tensor.rs:2241-2262)."""
    items = _items(array)
    toks = [("Struct", "Tensor", 2), ("Str", "dim"), ("Tuple", array.ndim)]
    toks += [("U64", int(d)) for d in array.shape]
    toks += [("TupleEnd",), ("Str", "buffer"), ("TupleStruct", "Buffer", 3), ("Str", scalar_name(array, bf16)),
             ("U64", int(array.size)), ("Seq", len(items))]
    toks += [("U64", v) for v in items]
    toks += [("SeqEnd",), ("TupleStructEnd",), ("StructEnd",)]
    return toks


def to_value(array, bf16=False):
    """The tensor as the JSON value serde_json writes: a struct is an object, tuples and tuple structs are arrays."""
    return {"dim": [int(d) for d in array.shape], "buffer": [scalar_name(array, bf16), int(array.size), _items(array)]}


def to_json(array, bf16=False):
    """What serde_json writes for the same value."""
    return json.dumps(to_value(array, bf16), separators=(",", ":"))


def from_json(text):
    """-> (array, is_bf16).  Rejects what the reference's `Deserialize` rejects: a missing or unknown field, a
    buffer whose length does not match, a `dim` whose product is not the element count (`into_shape`,
    src/tensor.rs:1245-1247)."""
    try:
        obj = json.loads(text)
    except json.JSONDecodeError as e:
        raise SerdeError(f"not JSON: {e}") from None
    return from_value(obj)


def from_value(obj):
    """`from_json` for an already parsed JSON value."""
    if not isinstance(obj, dict) or set(obj) != {"dim", "buffer"}:
        raise SerdeError("expected an object with exactly the fields `dim` and `buffer`")
    dim, buf = obj["dim"], obj["buffer"]
    if not isinstance(dim, list) or any(not isinstance(d, int) or isinstance(d, bool) or d < 0 for d in dim):
        raise SerdeError("`dim` must be an array of unsigned integers")
    if not isinstance(buf, list) or len(buf) != 3 or not isinstance(buf[0], str) or not isinstance(buf[1], int) \
            or isinstance(buf[1], bool) or buf[1] < 0 or not isinstance(buf[2], list):
        raise SerdeError("`buffer` must be [scalar type, length, items]")
    name, count, items = buf
    flat = _from_items(items, name, count)
    if int(np.prod(dim, dtype=np.int64)) != count:
        raise SerdeError(f"IncompatibleShape: dim {dim} does not hold {count} elements")
    return flat.reshape(dim), name == "BF16"


# ---- layers (src/learn/neural_network/layer.rs) ----
# The reference derives Serialize / Deserialize for its layer structs, so their data model is the field list:
#   Conv<D>    { weight: Parameter, padding: D, stride: D, dilation: D, bias: Option<Parameter1> }   (layer.rs:833-848)
#   Dense      { weight: Parameter2, bias: Option<Parameter1> }                                      (layer.rs:1069-1073)
#   MaxPool<D> { filter: D, stride: D }                                                              (layer.rs:1150-1155)
#   Relu, Flatten, Identity: unit structs (serde_json: null)                                        (layer.rs:1222-1252)
#   Parameter  { value: Tensor, optim_state }, `grad` skipped and `optim_state` skipped when it is none, absent ->
#              none (autograd.rs:639-656); ndarray's fixed-rank dimensions are tuples of integers.
# No vector of these is held by the reference's tests (its serde tests cover tensors only), so beyond the field
# names and order of the derive this encoding is unpinned; it is what serde_json makes of that data model.
# Values here are host arrays: (array, is_bf16) pairs as `from_value` returns them.


def _dims(obj, what, rank):
    if not isinstance(obj, list) or len(obj) != rank or any(not isinstance(d, int) or isinstance(d, bool) or d < 0 for d in obj):
        raise SerdeError(f"`{what}` must be an array of {rank} unsigned integers")
    return tuple(obj)


class OptimStateValue:
    """`State { name, id (skipped), key_values: Vec<(String, Value)> }` (optimizer.rs:163-173) on the host.
    `key_values`: [(key, array, is_bf16, parameter_device, parameter_type)]: every value a
    `Value::Tensor(TensorValue { tensor, parameter_device, parameter_type })` (optimizer.rs:108-131), the only kind
    the reference's optimizers create (SGD's "velocity", optimizer.rs:367-381)."""

    def __init__(self, name, key_values=()):
        self.name, self.key_values = str(name), [tuple(kv) for kv in key_values]


class ParamValue(tuple):
    """(array, is_bf16) of a parameter, with its optimizer state (None or an OptimStateValue) as `.optim_state`."""

    def __new__(cls, array, is_bf16, optim_state=None):
        self = super().__new__(cls, (array, is_bf16))
        self.optim_state = optim_state
        return self


def optim_state_to_value(state):
    return {"name": state.name,
            "key_values": [[str(key), {"Tensor": {"tensor": to_value(array, bf16), "parameter_device": bool(pdev),
                                                  "parameter_type": bool(ptype)}}]
                           for (key, array, bf16, pdev, ptype) in state.key_values]}


def optim_state_from_value(obj):
    # the derives set no `deny_unknown_fields`: keys they do not know are skipped, like serde's derive skips them
    if not isinstance(obj, dict) or not {"name", "key_values"} <= set(obj) or not isinstance(obj["name"], str) \
            or not isinstance(obj["key_values"], list):
        raise SerdeError("expected an optimizer state with the fields `name` and `key_values`")
    out = []
    for kv in obj["key_values"]:
        if not isinstance(kv, list) or len(kv) != 2 or not isinstance(kv[0], str) or not isinstance(kv[1], dict) \
                or len(kv[1]) != 1:
            raise SerdeError("`key_values` must hold [key, {variant: value}] pairs")
        (variant, value), = kv[1].items()
        if variant == "Elem":
            # the element type of Value::Elem is the scalar crate's, whose encoding no file of the reference holds
            raise SerdeError("optimizer state with a scalar element value is not supported here")
        if variant != "Tensor" or not isinstance(value, dict) or not {"tensor", "parameter_device", "parameter_type"} <= set(value) \
                or not isinstance(value["parameter_device"], bool) or not isinstance(value["parameter_type"], bool):
            raise SerdeError("expected {\"Tensor\": {tensor, parameter_device, parameter_type}}")
        array, is_bf16 = from_value(value["tensor"])
        out.append((kv[0], array, is_bf16, value["parameter_device"], value["parameter_type"]))
    return OptimStateValue(obj["name"], out)


def parameter_to_value(array, bf16=False, optim_state=None):
    """`value`, then `optim_state` unless it is none (skip_serializing_if, autograd.rs:651-655)."""
    out = {"value": to_value(array, bf16)}
    if optim_state is not None:
        out["optim_state"] = optim_state_to_value(optim_state)
    return out


def parameter_from_value(obj, rank):
    """-> ParamValue.  An absent `optim_state` is none (`default`); a present one must be a state: the reference's
    deserializer has no none case (autograd.rs:1141-1151)."""
    if not isinstance(obj, dict) or "value" not in obj:
        raise SerdeError("expected a parameter object with the field `value`")
    state = optim_state_from_value(obj["optim_state"]) if "optim_state" in obj else None
    array, is_bf16 = from_value(obj["value"])
    if array.ndim != rank:
        raise SerdeError(f"IncompatibleShape: a parameter of rank {rank} holds a tensor of rank {array.ndim}")
    return ParamValue(array, is_bf16, state)


def conv2_to_value(weight, bias=None, padding=(0, 0), stride=(1, 1), dilation=(1, 1), bf16=False, weight_state=None,
                   bias_state=None):
    return {"weight": parameter_to_value(weight, bf16, weight_state), "padding": [int(v) for v in padding],
            "stride": [int(v) for v in stride], "dilation": [int(v) for v in dilation],
            "bias": None if bias is None else parameter_to_value(bias, bf16, bias_state)}


def conv2_from_value(obj):
    """-> dict(weight=ParamValue, bias=None | ParamValue, padding, stride, dilation)"""
    # As the derive reads it (layer.rs:833-848, no `deny_unknown_fields`): unknown keys are skipped, a missing
    # `Option` field (`bias`) is None, any other missing field is an error.
    fields = {"weight", "padding", "stride", "dilation"}
    if not isinstance(obj, dict) or not fields <= set(obj):
        raise SerdeError("missing field: expected an object with the fields " + ", ".join(sorted(fields)) + " (and `bias`)")
    return dict(weight=parameter_from_value(obj["weight"], 4),
                bias=None if obj.get("bias") is None else parameter_from_value(obj["bias"], 1),
                padding=_dims(obj["padding"], "padding", 2), stride=_dims(obj["stride"], "stride", 2),
                dilation=_dims(obj["dilation"], "dilation", 2))


def dense_to_value(weight, bias=None, bf16=False, weight_state=None, bias_state=None):
    return {"weight": parameter_to_value(weight, bf16, weight_state),
            "bias": None if bias is None else parameter_to_value(bias, bf16, bias_state)}


def dense_from_value(obj):
    # layer.rs:1069-1073: a missing `bias` is None, unknown keys are skipped
    if not isinstance(obj, dict) or "weight" not in obj:
        raise SerdeError("missing field `weight`")
    return dict(weight=parameter_from_value(obj["weight"], 2),
                bias=None if obj.get("bias") is None else parameter_from_value(obj["bias"], 1))


def max_pool2_to_value(filter, stride):
    return {"filter": [int(v) for v in filter], "stride": [int(v) for v in stride]}


def max_pool2_from_value(obj):
    if not isinstance(obj, dict) or not {"filter", "stride"} <= set(obj):
        raise SerdeError("missing field: expected an object with the fields `filter` and `stride`")
    return dict(filter=_dims(obj["filter"], "filter", 2), stride=_dims(obj["stride"], "stride", 2))
