"""Abstract instruction executor: handler registry, buffer bookkeeping and
the instruction loop.

Same contract as the reference's ``dcp/core/executor.py`` (``DCPExecutor``
:33-198): handlers are callables ``handler(executor, instr)`` registered per
instruction type, every leaf subclass of ``BlockInstrBase`` must have one
(:158-178), buffers come from the plan's ``BufferInfo`` table (:106-126), and
a ``synchronous`` executor synchronises the device after each instruction
(:197-198).
"""

from __future__ import annotations

from typing import Any, Callable, Dict, Iterator, Optional, Tuple, Type

from dcp_amd.core.instructions import (
    BlockInstrBase,
    BufferType,
    ExecutionPlan,
)
from dcp_amd.utils.logger import create_logger, read_env_bool

DEBUG_LOG_EXECUTOR = read_env_bool("DCP_DEBUG_LOG_EXECUTOR", default=False)

# the padded slot buffers are scratch of one pass: dropped when the executor changes pass
_TMP_BUFFER_TYPES = frozenset(v for k, v in vars(BufferType).items() if k.startswith("BUFFER_"))

Handler = Callable[["DCPExecutor", BlockInstrBase], None]


def _leaves(root: Type[BlockInstrBase]) -> Iterator[Type[BlockInstrBase]]:
    children = root.__subclasses__()
    if not children:
        yield root
        return
    for child in children:
        yield from _leaves(child)


class HandlerTable:
    """Callables registered per leaf instruction type; ``what`` names the table in messages."""

    def __init__(self, what: str):
        self.what = what
        self._by_type: Dict[type, Handler] = {}

    def register(self, instruction_type, handler: Handler) -> None:
        if not (isinstance(instruction_type, type) and issubclass(instruction_type, BlockInstrBase)):
            raise TypeError(
                "Instruction type must be a subclass of BlockInstrBase, got "
                f"{getattr(instruction_type, '__name__', instruction_type)}"
            )
        if instruction_type in self._by_type:
            raise ValueError(f"{self.what} for {instruction_type.__name__} already registered.")
        self._by_type[instruction_type] = handler

    def get(self, instruction_type) -> Optional[Handler]:
        return self._by_type.get(instruction_type)

    def require(self, instruction_type) -> Handler:
        handler = self._by_type.get(instruction_type)
        if handler is None:
            raise ValueError(f"No handler registered for instruction {instruction_type.__name__}")
        return handler

    def __contains__(self, instruction_type) -> bool:
        return instruction_type in self._by_type


class DCPExecutor:
    """Runs one device's ``ExecutionPlan`` by dispatching each instruction to
    its registered handler."""

    def __init__(self, node_id: int = None, local_device_id: int = None, n_devices_per_node: int = None,
                 n_nodes: int = None, synchronous: bool = False, iteration_idx: Optional[int] = None,
                 tp_rank: Optional[int] = None):
        self.node_id, self.local_device_id = node_id, local_device_id
        self.n_devices_per_node, self.n_nodes = n_devices_per_node, n_nodes
        self.synchronous = synchronous
        self.tp_rank, self.iteration_idx = tp_rank, iteration_idx
        self.logger = None
        if DEBUG_LOG_EXECUTOR:
            tag = f"N{node_id}D{local_device_id}"
            suffix = (f"T{tp_rank}" if tp_rank is not None else "") + (f"_I{iteration_idx}" if iteration_idx is not None else "")
            self.logger = create_logger("DCPExecutor", prefix=tag, log_file=f"executor/{tag}{suffix}.log")
        self._handlers = HandlerTable("Instruction handler")
        self.instr_index = 0
        self.return_values: Dict[int, Any] = {}
        self.buffers: Dict[str, Any] = {}
        # per buffer type, from the plan's BufferInfo table: slots, elements per slot, tokens per
        # slot, shape of one token
        self.buffer_n_blocks: Dict[str, int] = {}
        self.buffer_block_strides: Dict[str, int] = {}
        self.buffer_block_sizes: Dict[str, int] = {}
        self.buffer_per_token_shape: Dict[str, Tuple[int, ...]] = {}

    # -- ranks: devices are numbered node by node ---------------------------------------
    def get_rank(self, node_id: int, local_device_id: int):
        return local_device_id + self.n_devices_per_node * node_id

    def reverse_get_rank(self, rank: int):
        return divmod(rank, self.n_devices_per_node)

    @property
    def rank(self):
        return self.get_rank(self.node_id, self.local_device_id)

    # -- buffers -------------------------------------------------------------
    def init_forward_input(self, local_q, local_kv):
        for buffer_type, value in ((BufferType.LOCAL_Q, local_q), (BufferType.LOCAL_KV, local_kv)):
            self.buffers[buffer_type].copy_(value)

    def init_backward_input(self, local_dout):
        self.buffers[BufferType.LOCAL_dOUT].copy_(local_dout)

    def deallocate_buffers(self):
        """Drop the padded slot buffers (the caller-facing LOCAL_* buffers stay)."""
        for buffer_type in _TMP_BUFFER_TYPES & set(self.buffers):
            self.buffers[buffer_type] = None

    def init_buffers(self, execution_plan: ExecutionPlan):
        for buffer_type, info in execution_plan.buffer_info.items():
            self.buffer_n_blocks[buffer_type] = info.n_blocks
            self.buffer_block_strides[buffer_type] = info.block_numel
            self.buffer_block_sizes[buffer_type] = info.block_size
            self.buffer_per_token_shape[buffer_type] = info.per_token_shape
            if self.buffers.get(buffer_type) is not None:
                continue
            if self.logger:
                self.logger.debug("Creating buffer %s shape %s dtype %s per-token %s", buffer_type,
                                  info.buffer_shape, info.dtype, info.per_token_shape)
            self.buffers[buffer_type] = self._create_buffer(info.buffer_shape, info.dtype)

    def _create_buffer(self, buffer_shape: Tuple[int, ...], buffer_dtype: int):
        raise NotImplementedError("DCPExecutor._create_buffer not implemented")

    # -- handler registry ----------------------------------------------------
    def register_handler(self, instruction_type, handler: Handler):
        self._handlers.register(instruction_type, handler)

    @classmethod
    def _get_leaf_subclasses(cls, instruction_type: Type[BlockInstrBase]):
        return _leaves(instruction_type)

    @classmethod
    def get_all_needed_handlers(cls):
        return sorted({t.__name__ for t in _leaves(BlockInstrBase)})

    def check_all_handlers_registered(self):
        for instruction_type in _leaves(BlockInstrBase):
            self._handlers.require(instruction_type)

    def register_synchronization_handler(self, handler):
        self.synchronize = handler

    def synchronize(self):
        raise NotImplementedError("Synchronization handler not registered")

    # -- the loop ------------------------------------------------------------
    def execute(self, execution_plan: ExecutionPlan, is_forward: bool = True):
        self.execution_plan = execution_plan
        self.init_buffers(execution_plan)
        for self.instr_index, instruction in enumerate(execution_plan.instructions):
            if self.logger:
                self.logger.debug("Executing instruction: %s", instruction)
            self._execute_instruction(instruction)
        if self.logger:
            self.logger.debug("Execution complete.")
        return self.return_values

    def _execute_instruction(self, instruction: BlockInstrBase):
        self._handlers.require(type(instruction))(self, instruction)
        if self.synchronous:
            self.synchronize()
