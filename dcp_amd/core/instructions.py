"""Block-instruction data model consumed by the executor.

Mirrors the types, field names, opcode numbering and wire format of the
reference's ``dcp/core/instructions.py`` (``BufferType`` :21-37, ``DType``
:63-106, ``BufferBlock`` :184-198, ``MemcpyInstr`` :303-344, comm instructions
:347-476, ``AttnInstr`` :500-626, ``AttnBackwardInstr`` :629-746,
``ReductionOp``/``AttnReductionInstr`` :749-833, ``SumOp``/``SumInstr``
:836-907, ``BufferInfo`` :910-917, ``ExecutionPlan`` :920-1079) so a plan built
for the reference executor drives this one unchanged.

The implementation is declarative: every instruction lists its fields with a
codec, and one generic encoder/decoder walks that list.  Opcodes are the
definition order of the ``BlockInstrBase`` subclasses, which therefore must
stay: Memcpy, CommLaunch, Barrier, CommWait, Attn, AttnBackward,
AttnReduction, Sum.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Optional, Sequence, Tuple, Type

import numpy as np
import torch

from dcp_amd.core.serialization import (
    ByteReader,
    ByteWriter,
    SerializationConfig,
)


class BufferType:
    # persistent, unpadded, token-major buffers owned by the caller's layout
    LOCAL_Q = "LocalQ"
    LOCAL_KV = "LocalKV"
    LOCAL_dQ = "LocaldQ"
    LOCAL_dKV = "LocaldKV"
    LOCAL_OUT = "LocalOut"
    LOCAL_dOUT = "LocaldOut"
    LOCAL_LSE = "LocalLSE"
    # padded slot buffers the kernels page through
    BUFFER_Q = "BufferQ"
    BUFFER_KV = "BufferKV"
    BUFFER_dQ = "BufferdQ"
    BUFFER_dKV = "BufferdKV"
    BUFFER_OUT = "BufferOut"
    BUFFER_dOUT = "BufferdOut"
    BUFFER_LSE = "BufferLSE"


class CommType:
    SEND = 0
    RECV = 1

    @classmethod
    def from_num(cls, num):
        if num not in (cls.SEND, cls.RECV):
            raise ValueError(f"Invalid comm type {num}")
        return num

    @classmethod
    def to_str(cls, comm_type):
        try:
            return {cls.SEND: "send", cls.RECV: "recv"}[comm_type]
        except KeyError:
            raise ValueError(f"Invalid comm type {comm_type}") from None


class DType:
    BFLOAT16 = 0
    FLOAT16 = 1
    FLOAT32 = 2
    INT = 3

    _NAMES = {0: "bf16", 1: "fp16", 2: "fp32", 3: "int"}
    _SIZES = {0: 2, 1: 2, 2: 4, 3: 4}

    @classmethod
    def from_num(cls, num):
        if num not in cls._NAMES:
            raise ValueError(f"Invalid dtype {num}")
        return num

    @classmethod
    def as_str(cls, dtype):
        if dtype not in cls._NAMES:
            raise ValueError(f"Invalid dtype {dtype}")
        return cls._NAMES[dtype]

    @classmethod
    def element_size(cls, dtype):
        if dtype not in cls._SIZES:
            raise ValueError(f"Invalid dtype {dtype}")
        return cls._SIZES[dtype]


@dataclass(frozen=True)
class BufferBlock:
    """One block of a buffer: ``index`` is the slot (padded buffers) or the
    position in ``local_cu_seqlens`` (unpadded LOCAL_* buffers)."""

    buffer_type: str
    index: int
    n_tokens: int

    def __post_init__(self):
        assert self.buffer_type is not None
        assert isinstance(self.index, int)
        assert isinstance(self.n_tokens, int)

    def __repr__(self):
        return f"({self.buffer_type}, {self.index}, {self.n_tokens})"


# ---------------------------------------------------------------------------
# Field codecs: (encode(writer, value), decode(reader) -> value, equal(a, b))
# ---------------------------------------------------------------------------


@dataclass(frozen=True)
class _Codec:
    put: Callable[[ByteWriter, Any], None]
    get: Callable[[ByteReader], Any]
    same: Callable[[Any, Any], bool] = lambda a, b: a == b


def _put_block(w: ByteWriter, b: BufferBlock) -> None:
    w.string(b.buffer_type).uint(b.index).uint(b.n_tokens)


def _get_block(r: ByteReader) -> BufferBlock:
    return BufferBlock(r.string(), r.uint(), r.uint())


def _put_blocks(w: ByteWriter, blocks: Sequence[BufferBlock]) -> None:
    w.uint(len(blocks))
    for b in blocks:
        _put_block(w, b)


def _get_blocks(r: ByteReader) -> List[BufferBlock]:
    return [_get_block(r) for _ in range(r.uint())]


def _put_table(w: ByteWriter, table: Sequence[Sequence[BufferBlock]]) -> None:
    w.uint(len(table))
    for row in table:
        _put_blocks(w, row)


def _get_table(r: ByteReader) -> List[List[BufferBlock]]:
    return [_get_blocks(r) for _ in range(r.uint())]


def _mask_planes(mask) -> List[torch.Tensor]:
    """An attention mask travels as its leading-axis planes: 2 planes of [T]
    (one range per token) or 2 planes of [2, T] (two ranges)."""
    if isinstance(mask, torch.Tensor):
        return [mask[i] for i in range(mask.shape[0])]
    return list(mask)


def _put_mask(w: ByteWriter, mask) -> None:
    planes = _mask_planes(mask)
    w.uint(len(planes))
    for plane in planes:
        assert plane.dtype == torch.int32, "attention ranges must be int32"
        blob = plane.detach().cpu().contiguous().numpy().tobytes()
        w.uints(tuple(plane.shape)).uint(len(blob)).raw(blob)


def _get_mask(r: ByteReader) -> torch.Tensor:
    planes = []
    for _ in range(r.uint()):
        shape = tuple(r.uints())
        blob = r.raw(r.uint())
        arr = np.frombuffer(blob, dtype="<i4").reshape(shape).copy()
        planes.append(torch.from_numpy(arr))
    return torch.stack(planes, dim=0) if planes else torch.zeros(0, dtype=torch.int32)


def _same_mask(a, b) -> bool:
    pa, pb = _mask_planes(a), _mask_planes(b)
    return len(pa) == len(pb) and all(
        x.shape == y.shape and torch.equal(x, y) for x, y in zip(pa, pb)
    )


def _put_pairs(w: ByteWriter, pairs) -> None:
    w.uint(len(pairs))
    for src, dst in pairs:
        _put_block(w, src)
        _put_block(w, dst)


def _get_pairs(r: ByteReader):
    return [(_get_block(r), _get_block(r)) for _ in range(r.uint())]


def _opt_string(r: ByteReader):
    s = r.string()
    return s if s != "" else None


UINT = _Codec(lambda w, v: w.uint(int(v)), lambda r: r.uint())
UINTS = _Codec(lambda w, v: w.uints(v), lambda r: r.uints())
STRING = _Codec(lambda w, v: w.string(v), lambda r: r.string())
OPT_STRING = _Codec(lambda w, v: w.string(v), _opt_string)
BLOCK_TABLE = _Codec(_put_table, _get_table)
BLOCK_PAIRS = _Codec(_put_pairs, _get_pairs)
RANGE_MASK = _Codec(_put_mask, _get_mask, _same_mask)


class BlockInstrBase:
    """Base of all instructions.  Keyword arguments become attributes and are
    kept in ``kwargs`` for ``repr`` and equality."""

    _instr_index_to_cls: Dict[int, Type["BlockInstrBase"]] = {}
    _fields: Tuple[Tuple[str, _Codec], ...] = ()

    def __init__(self, **kwargs):
        self.name = type(self).__name__
        self.kwargs = kwargs
        for key, val in kwargs.items():
            setattr(self, key, val)

    def __init_subclass__(cls) -> None:
        cls._instr_index = len(BlockInstrBase._instr_index_to_cls)
        BlockInstrBase._instr_index_to_cls[cls._instr_index] = cls

    def __repr__(self):
        body = ", ".join(f"{k}={v!r}" for k, v in self.kwargs.items())
        return f"{self.name}({body})"

    def __eq__(self, other):
        if type(self) is not type(other):
            return False
        if not self._fields:
            return self.kwargs == other.kwargs
        return all(
            codec.same(getattr(self, name), getattr(other, name))
            for name, codec in self._fields
        )

    __hash__ = None

    def serialize(self, config=SerializationConfig()) -> bytes:
        w = ByteWriter(config).opcode(self._instr_index)
        for name, codec in self._fields:
            codec.put(w, getattr(self, name))
        return bytes(w)

    @classmethod
    def _read(cls, r: ByteReader) -> "BlockInstrBase":
        target = BlockInstrBase._instr_index_to_cls[r.opcode()]
        return target(**{name: codec.get(r) for name, codec in target._fields})

    @classmethod
    def deserialize(
        cls, data: bytes, config=SerializationConfig()
    ) -> Tuple["BlockInstrBase", bytes]:
        r = ByteReader(data, config)
        instr = cls._read(r)
        return instr, r.rest()


# --- opcode 0 --------------------------------------------------------------
class MemcpyInstr(BlockInstrBase):
    """Copy token blocks between buffers (gather LOCAL_* -> BUFFER_*)."""

    _fields = (("src_dst_pairs", BLOCK_PAIRS),)

    def __init__(
        self, src_dst_pairs: List[Tuple[BufferBlock, BufferBlock]], **kwargs
    ):
        super().__init__(src_dst_pairs=src_dst_pairs, **kwargs)
        self.src_dst_pairs: List[Tuple[BufferBlock, BufferBlock]]


@dataclass(frozen=True)
class CommOp:
    comm_type: int
    peer: Tuple[int, int]
    buffer_block: BufferBlock

    def _put(self, w: ByteWriter) -> None:
        w.uint(self.comm_type).uint(self.peer[0]).uint(self.peer[1])
        _put_block(w, self.buffer_block)

    @staticmethod
    def _get(r: ByteReader) -> "CommOp":
        comm_type = CommType.from_num(r.uint())
        peer = (r.uint(), r.uint())
        return CommOp(comm_type, peer, _get_block(r))

    def serialize(self, config=SerializationConfig()) -> bytes:
        w = ByteWriter(config)
        self._put(w)
        return bytes(w)

    def __repr__(self) -> str:
        return (
            f"CommOp(comm_type={CommType.to_str(self.comm_type)}, "
            f"peer={self.peer}, buffer_block={self.buffer_block})"
        )


def _put_comm_ops(w: ByteWriter, ops: Sequence[CommOp]) -> None:
    w.uint(len(ops))
    for op in ops:
        op._put(w)


COMM_OPS = _Codec(
    _put_comm_ops, lambda r: [CommOp._get(r) for _ in range(r.uint())]
)


# --- opcode 1 --------------------------------------------------------------
class CommLaunchInstr(BlockInstrBase):
    _fields = (("key", STRING), ("comm_ops", COMM_OPS), ("stream", OPT_STRING))

    def __init__(
        self,
        key: str,
        comm_ops: List[CommOp],
        stream: Optional[str] = None,
        **kwargs,
    ):
        super().__init__(key=key, comm_ops=comm_ops, stream=stream, **kwargs)


# --- opcode 2 --------------------------------------------------------------
class BarrierInstr(BlockInstrBase):
    pass


# --- opcode 3 --------------------------------------------------------------
class CommWaitInstr(BlockInstrBase):
    _fields = (("key", STRING), ("stream", OPT_STRING))

    def __init__(self, key: str, stream: Optional[str] = None, **kwargs):
        super().__init__(key=key, stream=stream, **kwargs)


def _table_repr(table: Sequence[Sequence[BufferBlock]]) -> str:
    if not table or not table[0]:
        return "[]"
    rows = ", ".join(
        "[" + ", ".join(str(b.index) for b in row) + "]" for row in table
    )
    return f"{table[0][0].buffer_type}[{rows}]"


_ATTN_COMMON = (
    ("stage_id", UINT),
    ("seqlens_q", UINTS),
    ("seqlens_kv", UINTS),
    ("max_seqlen_q", UINT),
    ("max_seqlen_kv", UINT),
    ("attn_mask", RANGE_MASK),
    ("q_block_table", BLOCK_TABLE),
    ("kv_block_table", BLOCK_TABLE),
    ("out_block_table", BLOCK_TABLE),
)


class _AttnReprMixin:
    def __repr__(self) -> str:
        parts = []
        for name, codec in self._fields:
            if codec is RANGE_MASK:
                continue
            value = getattr(self, name)
            if codec is BLOCK_TABLE:
                value = _table_repr(value)
            parts.append(f"{name}={value}")
        return f"{type(self).__name__}(" + ", ".join(parts) + ")"


# --- opcode 4 --------------------------------------------------------------
class AttnInstr(_AttnReprMixin, BlockInstrBase):
    """Range-masked paged attention forward.

    Batch row ``b`` is one q block: ``seqlens_q[b]`` query tokens read from
    ``q_block_table[b][0]``, attending over the concatenation of the blocks
    in ``kv_block_table[b]``.  ``attn_mask`` is int32 ``[2, sum(seqlens_q)]``
    (``[start, end)`` per query token, in the row's concatenated-kv
    coordinates) or ``[2, 2, sum(seqlens_q)]`` (two ranges; axis 0 is the
    range, axis 1 start/end); a token attends to the union.  The partial
    output and its log-sum-exp go to ``out_block_table[b][0]`` /
    ``lse_block_table[b][0]`` (same slot index).
    """

    _fields = _ATTN_COMMON + (("lse_block_table", BLOCK_TABLE),)

    def __init__(
        self,
        stage_id: int,
        seqlens_q: List[int],
        seqlens_kv: List[int],
        max_seqlen_q: int,
        max_seqlen_kv: int,
        attn_mask,
        q_block_table: List[List[BufferBlock]],
        kv_block_table: List[List[BufferBlock]],
        out_block_table: List[List[BufferBlock]],
        lse_block_table: List[List[BufferBlock]],
        **kwargs,
    ):
        super().__init__(
            stage_id=stage_id,
            seqlens_q=seqlens_q,
            seqlens_kv=seqlens_kv,
            max_seqlen_q=max_seqlen_q,
            max_seqlen_kv=max_seqlen_kv,
            attn_mask=attn_mask,
            q_block_table=q_block_table,
            kv_block_table=kv_block_table,
            out_block_table=out_block_table,
            lse_block_table=lse_block_table,
            **kwargs,
        )
        for out_row, lse_row in zip(out_block_table, lse_block_table):
            assert [b.index for b in out_row] == [b.index for b in lse_row]


# --- opcode 5 --------------------------------------------------------------
class AttnBackwardInstr(_AttnReprMixin, BlockInstrBase):
    """Range-masked paged attention backward.

    Rows as in :class:`AttnInstr`.  Out, LSE and dOut of a row share the slot
    index ``out_block_table[b][0]``.  dQ of the row accumulates into
    ``dq_block_table[b][0]``; ``dkv_block_table[b][j]`` is a private dKV block
    for the j-th kv block of the row (nothing is accumulated across rows).
    """

    _fields = _ATTN_COMMON + (
        ("dq_block_table", BLOCK_TABLE),
        ("dkv_block_table", BLOCK_TABLE),
    )

    def __init__(
        self,
        stage_id: int,
        seqlens_q: List[int],
        seqlens_kv: List[int],
        max_seqlen_q: int,
        max_seqlen_kv: int,
        attn_mask,
        q_block_table: List[List[BufferBlock]],
        kv_block_table: List[List[BufferBlock]],
        out_block_table: List[List[BufferBlock]],
        dq_block_table: List[List[BufferBlock]],
        dkv_block_table: List[List[BufferBlock]],
        **kwargs,
    ):
        super().__init__(
            stage_id=stage_id,
            seqlens_q=seqlens_q,
            seqlens_kv=seqlens_kv,
            max_seqlen_q=max_seqlen_q,
            max_seqlen_kv=max_seqlen_kv,
            attn_mask=attn_mask,
            q_block_table=q_block_table,
            kv_block_table=kv_block_table,
            out_block_table=out_block_table,
            dq_block_table=dq_block_table,
            dkv_block_table=dkv_block_table,
            **kwargs,
        )


@dataclass
class ReductionOp:
    """Merge the (out, lse) partials in ``src_buffers`` into ``dst_buffer``."""

    src_buffers: List[Tuple[BufferBlock, BufferBlock]]
    dst_buffer: Tuple[BufferBlock, BufferBlock]

    def __post_init__(self):
        assert self.dst_buffer[0].index == self.dst_buffer[1].index
        for src_out, src_lse in self.src_buffers:
            if src_out.index != src_lse.index:
                raise ValueError(
                    "src_out and src_lse buffer indices do not match: "
                    f"{src_out.index} != {src_lse.index}"
                )

    def _put(self, w: ByteWriter) -> None:
        _put_pairs(w, self.src_buffers)
        _put_block(w, self.dst_buffer[0])
        _put_block(w, self.dst_buffer[1])

    @staticmethod
    def _get(r: ByteReader) -> "ReductionOp":
        srcs = _get_pairs(r)
        return ReductionOp(srcs, (_get_block(r), _get_block(r)))

    def serialize(self, config=SerializationConfig()) -> bytes:
        w = ByteWriter(config)
        self._put(w)
        return bytes(w)


def _ops_codec(op_type) -> _Codec:
    def put(w: ByteWriter, ops) -> None:
        w.uint(len(ops))
        for op in ops:
            op._put(w)

    return _Codec(put, lambda r: [op_type._get(r) for _ in range(r.uint())])


# --- opcode 6 --------------------------------------------------------------
class AttnReductionInstr(BlockInstrBase):
    """N-way online-softmax merge; ``output_is_unpadded`` selects whether the
    destination is a LOCAL_* buffer addressed by ``local_cu_seqlens`` (1) or a
    padded slot (0)."""

    _fields = (
        ("ops", _ops_codec(ReductionOp)),
        ("output_is_unpadded", UINT),
    )

    def __init__(self, ops: List[ReductionOp], output_is_unpadded: int, **kwargs):
        super().__init__(
            ops=ops, output_is_unpadded=output_is_unpadded, **kwargs
        )


@dataclass
class SumOp:
    """Element-wise sum of ``src_buffers`` into ``dst_buffer``."""

    src_buffers: List[BufferBlock]
    dst_buffer: BufferBlock

    def _put(self, w: ByteWriter) -> None:
        _put_blocks(w, self.src_buffers)
        _put_block(w, self.dst_buffer)

    @staticmethod
    def _get(r: ByteReader) -> "SumOp":
        return SumOp(_get_blocks(r), _get_block(r))

    def serialize(self, config=SerializationConfig()) -> bytes:
        w = ByteWriter(config)
        self._put(w)
        return bytes(w)


# --- opcode 7 --------------------------------------------------------------
class SumInstr(BlockInstrBase):
    _fields = (("ops", _ops_codec(SumOp)), ("output_is_unpadded", UINT))

    def __init__(self, ops: List[SumOp], output_is_unpadded: int, **kwargs):
        super().__init__(
            ops=ops, output_is_unpadded=output_is_unpadded, **kwargs
        )


@dataclass
class BufferInfo:
    n_blocks: int
    block_size: int  # tokens per (padded) block
    block_numel: int  # elements per padded block
    dtype: int  # wire dtype integer, see serialization.int_to_torch_dtype
    buffer_shape: Tuple[int, ...]
    per_token_shape: Tuple[int, ...]


class ExecutionPlan:
    """The instruction list of one device plus the buffers it runs over."""

    _META = (
        "n_nodes",
        "n_devices_per_node",
        "node_id",
        "local_device_id",
        "n_stages",
    )

    def __init__(
        self,
        instructions: List[BlockInstrBase],
        n_nodes: int,
        n_devices_per_node: int,
        node_id: int,
        local_device_id: int,
        n_stages: int,
        local_cu_seqlens: List[int],
        buffer_info: Dict[str, BufferInfo],
    ):
        self.instructions = instructions
        self.n_nodes = n_nodes
        self.n_devices_per_node = n_devices_per_node
        self.node_id = node_id
        self.local_device_id = local_device_id
        self.n_stages = n_stages
        self.local_cu_seqlens = local_cu_seqlens
        self.buffer_info = buffer_info

    def _header(self) -> str:
        meta = ", ".join(f"{k}={getattr(self, k)}" for k in self._META)
        return (
            f"ExecutionPlan({meta}, buffer_info={self.buffer_info}, "
            f"local_cu_seqlens={self.local_cu_seqlens}"
        )

    def __repr__(self) -> str:
        return f"{self._header()}, instructions={self.instructions})"

    def __str__(self) -> str:
        body = "\n\t".join(str(x) for x in self.instructions)
        return f"{self._header()}, instructions=[\n\t{body}\n])"

    def __eq__(self, other):
        if not isinstance(other, ExecutionPlan):
            return False
        return (
            all(getattr(self, k) == getattr(other, k) for k in self._META)
            and self.buffer_info == other.buffer_info
            and self.local_cu_seqlens == other.local_cu_seqlens
            and self.instructions == other.instructions
        )

    __hash__ = None

    def _put(self, w: ByteWriter) -> None:
        for k in self._META:
            w.uint(getattr(self, k))
        w.uints(self.local_cu_seqlens)
        w.uint(len(self.buffer_info))
        for name, info in self.buffer_info.items():
            w.string(name).uint(info.n_blocks).uint(info.block_size)
            w.uint(info.block_numel).uint(info.dtype)
            w.uints(tuple(info.buffer_shape)).uints(tuple(info.per_token_shape))
        w.uint(len(self.instructions))
        for instr in self.instructions:
            w.raw(instr.serialize(w.config))

    @classmethod
    def _get(cls, r: ByteReader) -> "ExecutionPlan":
        meta = {k: r.uint() for k in cls._META}
        local_cu_seqlens = r.uints()
        buffer_info = {}
        for _ in range(r.uint()):
            name = r.string()
            n_blocks, block_size = r.uint(), r.uint()
            block_numel, dtype = r.uint(), r.uint()
            shape, per_token = tuple(r.uints()), tuple(r.uints())
            buffer_info[name] = BufferInfo(
                n_blocks, block_size, block_numel, dtype, shape, per_token
            )
        instructions = [BlockInstrBase._read(r) for _ in range(r.uint())]
        return cls(
            instructions,
            local_cu_seqlens=local_cu_seqlens,
            buffer_info=buffer_info,
            **meta,
        )

    def serialize(self, config=SerializationConfig()) -> bytes:
        w = ByteWriter(config)
        self._put(w)
        return bytes(w)

    @classmethod
    def deserialize(
        cls, data: bytes, config=SerializationConfig()
    ) -> Tuple["ExecutionPlan", bytes]:
        r = ByteReader(data, config)
        plan = cls._get(r)
        return plan, r.rest()


def serialize_list_of_execution_plans(
    execution_plans: List[ExecutionPlan], config=SerializationConfig()
) -> bytes:
    w = ByteWriter(config).uint(len(execution_plans))
    for plan in execution_plans:
        plan._put(w)
    return bytes(w)


def deserialize_list_of_execution_plans(
    data: bytes, config=SerializationConfig()
) -> Tuple[List[ExecutionPlan], bytes]:
    r = ByteReader(data, config)
    plans = [ExecutionPlan._get(r) for _ in range(r.uint())]
    return plans, r.rest()
