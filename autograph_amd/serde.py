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


def to_json(array, bf16=False):
    """What serde_json writes for the same value: a struct is an object, tuples and tuple structs are arrays."""
    return json.dumps({"dim": [int(d) for d in array.shape],
                       "buffer": [scalar_name(array, bf16), int(array.size), _items(array)]}, separators=(",", ":"))


def from_json(text):
    """-> (array, is_bf16).  Rejects what the reference's `Deserialize` rejects: a missing or unknown field, a
    buffer whose length does not match, a `dim` whose product is not the element count (`into_shape`,
    src/tensor.rs:1245-1247)."""
    try:
        obj = json.loads(text)
    except json.JSONDecodeError as e:
        raise SerdeError(f"not JSON: {e}") from None
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
