"""Wire codecs for execution plans.

Every integer is an unsigned little-endian field of ``EXECUTION_PLAN_META_BYTES``
(4) bytes, an opcode is ``INSTRUCTION_INDEX_BYTES`` (1) byte, a string is a
length-prefixed UTF-8 run (an empty or ``None`` string is a bare zero length),
a float is an 8-byte little-endian double.  The byte layout follows the
reference's ``dcp/core/serialization.py:10-120`` so that plans produced by a
reference planner decode here; the implementation is built on ``struct`` and a
cursor instead of slicing the tail of the buffer on every field.

The function names of the reference (``int_meta_to_bytes`` ...) are kept as
the public API: each decoder returns ``(value, remaining_bytes)``.
"""

from __future__ import annotations

import struct
from dataclasses import dataclass
from typing import Dict, Iterable, List, Sequence, Tuple

import torch


@dataclass
class SerializationConfig:
    BYTES_ENDIANNESS = "little"
    FLOAT_BYTES_ENDIANNESS = "<"
    INSTRUCTION_INDEX_BYTES = 1
    EXECUTION_PLAN_META_BYTES = 4


_DEFAULT = SerializationConfig()


def _int_fmt(config: SerializationConfig, count: int = 1) -> str:
    width = config.EXECUTION_PLAN_META_BYTES
    code = {1: "B", 2: "H", 4: "I", 8: "Q"}[width]
    order = "<" if config.BYTES_ENDIANNESS == "little" else ">"
    return f"{order}{count}{code}"


class ByteWriter:
    """Append-only encoder; ``bytes(writer)`` yields the encoded buffer."""

    def __init__(self, config: SerializationConfig = _DEFAULT):
        self.config = config
        self._parts: List[bytes] = []

    def opcode(self, index: int) -> "ByteWriter":
        self._parts.append(
            index.to_bytes(
                self.config.INSTRUCTION_INDEX_BYTES,
                self.config.BYTES_ENDIANNESS,
            )
        )
        return self

    def uint(self, value: int) -> "ByteWriter":
        self._parts.append(struct.pack(_int_fmt(self.config), value))
        return self

    def uints(self, values: Sequence[int]) -> "ByteWriter":
        """Length-prefixed run of integers."""
        values = list(values)
        self._parts.append(
            struct.pack(
                _int_fmt(self.config, len(values) + 1), len(values), *values
            )
        )
        return self

    def string(self, value) -> "ByteWriter":
        raw = value.encode() if value else b""
        self.uint(len(raw))
        self._parts.append(raw)
        return self

    def double(self, value: float) -> "ByteWriter":
        self._parts.append(
            struct.pack(self.config.FLOAT_BYTES_ENDIANNESS + "d", value)
        )
        return self

    def raw(self, blob: bytes) -> "ByteWriter":
        self._parts.append(bytes(blob))
        return self

    def __bytes__(self) -> bytes:
        return b"".join(self._parts)


class ByteReader:
    """Cursor over an encoded buffer (no copies until ``rest()``)."""

    def __init__(self, data, config: SerializationConfig = _DEFAULT):
        self.config = config
        self._view = memoryview(bytes(data))
        self._pos = 0

    def _take(self, n: int) -> memoryview:
        end = self._pos + n
        if end > len(self._view):
            raise ValueError(
                f"truncated buffer: need {n} bytes at offset {self._pos}, "
                f"have {len(self._view) - self._pos}"
            )
        chunk = self._view[self._pos : end]
        self._pos = end
        return chunk

    def opcode(self) -> int:
        return int.from_bytes(
            self._take(self.config.INSTRUCTION_INDEX_BYTES),
            self.config.BYTES_ENDIANNESS,
        )

    def uint(self) -> int:
        width = self.config.EXECUTION_PLAN_META_BYTES
        return struct.unpack(_int_fmt(self.config), self._take(width))[0]

    def uints(self) -> List[int]:
        n = self.uint()
        width = self.config.EXECUTION_PLAN_META_BYTES
        return list(
            struct.unpack(_int_fmt(self.config, n), self._take(n * width))
        )

    def string(self) -> str:
        n = self.uint()
        return bytes(self._take(n)).decode() if n else ""

    def double(self) -> float:
        return struct.unpack(
            self.config.FLOAT_BYTES_ENDIANNESS + "d", self._take(8)
        )[0]

    def raw(self, n: int) -> bytes:
        return bytes(self._take(n))

    def rest(self) -> bytes:
        return bytes(self._view[self._pos :])


# ---------------------------------------------------------------------------
# Function API (names and return conventions of the reference module).
# ---------------------------------------------------------------------------


def int_meta_to_bytes(n: int, config=_DEFAULT) -> bytes:
    return bytes(ByteWriter(config).uint(n))


def bytes_to_int_meta(data: bytes, config=_DEFAULT) -> Tuple[int, bytes]:
    r = ByteReader(data, config)
    return r.uint(), r.rest()


def serialize_list_of_ints(ints: Iterable[int], config=_DEFAULT) -> bytes:
    return bytes(ByteWriter(config).uints(list(ints)))


def deserialize_list_of_ints(data, config=_DEFAULT) -> Tuple[List[int], bytes]:
    r = ByteReader(data, config)
    return r.uints(), r.rest()


def serialize_int_tuple(t: Tuple[int, ...], config=_DEFAULT) -> bytes:
    return bytes(ByteWriter(config).uints(tuple(int(x) for x in t)))


def deserialize_int_tuple(
    data, config=_DEFAULT
) -> Tuple[Tuple[int, ...], bytes]:
    r = ByteReader(data, config)
    return tuple(r.uints()), r.rest()


def serialize_str(s, config=_DEFAULT) -> bytes:
    return bytes(ByteWriter(config).string(s))


def deserialize_str(data, config=_DEFAULT) -> Tuple[str, bytes]:
    r = ByteReader(data, config)
    return r.string(), r.rest()


def serialize_float(f: float, config=_DEFAULT) -> bytes:
    return bytes(ByteWriter(config).double(f))


def deserialize_float(data, config=_DEFAULT) -> Tuple[float, bytes]:
    r = ByteReader(data, config)
    return r.double(), r.rest()


def serialize_list_of_floats(floats, config=_DEFAULT) -> bytes:
    w = ByteWriter(config).uint(len(floats))
    for f in floats:
        w.double(f)
    return bytes(w)


def deserialize_list_of_floats(data, config=_DEFAULT):
    r = ByteReader(data, config)
    return [r.double() for _ in range(r.uint())], r.rest()


def serialize_list_of_list_of_ints(lists, config=_DEFAULT) -> bytes:
    w = ByteWriter(config).uint(len(lists))
    for inner in lists:
        w.uints(inner)
    return bytes(w)


def deserialize_list_of_list_of_ints(data, config=_DEFAULT):
    r = ByteReader(data, config)
    return [r.uints() for _ in range(r.uint())], r.rest()


def serialize_dict_of_int_to_int(d: Dict[int, int], config=_DEFAULT) -> bytes:
    w = ByteWriter(config).uint(len(d))
    for k, v in d.items():
        w.uint(k).uint(v)
    return bytes(w)


def deserialize_dict_of_int_to_int(data, config=_DEFAULT):
    r = ByteReader(data, config)
    out = {}
    for _ in range(r.uint()):
        k = r.uint()
        out[k] = r.uint()
    return out, r.rest()


# torch dtype <-> wire integer (reference serialization.py:410-437).
_TORCH_DTYPES = (
    torch.bfloat16,
    torch.float16,
    torch.float32,
    torch.int32,
    torch.int64,
)


def torch_dtype_to_int(dtype: torch.dtype) -> int:
    try:
        return _TORCH_DTYPES.index(dtype)
    except ValueError:
        raise ValueError(f"Unsupported dtype: {dtype}") from None


def int_to_torch_dtype(dtype: int) -> torch.dtype:
    if not 0 <= dtype < len(_TORCH_DTYPES):
        raise ValueError(f"Unsupported dtype: {dtype}")
    return _TORCH_DTYPES[dtype]
