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

_LOCAL_BUFFER_TYPES_FW = (BufferType.LOCAL_Q, BufferType.LOCAL_KV)
_LOCAL_BUFFER_TYPES_BW = _LOCAL_BUFFER_TYPES_FW + (
    BufferType.LOCAL_OUT,
    BufferType.LOCAL_LSE,
    BufferType.LOCAL_dOUT,
)
_TMP_BUFFER_TYPES = frozenset(
    (
        BufferType.BUFFER_Q,
        BufferType.BUFFER_KV,
        BufferType.BUFFER_OUT,
        BufferType.BUFFER_LSE,
        BufferType.BUFFER_dOUT,
        BufferType.BUFFER_dQ,
        BufferType.BUFFER_dKV,
    )
)

Handler = Callable[["DCPExecutor", BlockInstrBase], None]


def _leaves(root: Type[BlockInstrBase]) -> Iterator[Type[BlockInstrBase]]:
    children = root.__subclasses__()
    if not children:
        yield root
        return
    for child in children:
        yield from _leaves(child)


class DCPExecutor:
    """Runs one device's ``ExecutionPlan`` by dispatching each instruction to
    its registered handler."""

    def __init__(
        self,
        node_id: int = None,
        local_device_id: int = None,
        n_devices_per_node: int = None,
        n_nodes: int = None,
        synchronous: bool = False,
        iteration_idx: Optional[int] = None,
        tp_rank: Optional[int] = None,
    ):
        self.node_id = node_id
        self.local_device_id = local_device_id
        self.n_devices_per_node = n_devices_per_node
        self.n_nodes = n_nodes
        self.synchronous = synchronous
        self.tp_rank = tp_rank
        self.iteration_idx = iteration_idx
        self.logger = None
        if DEBUG_LOG_EXECUTOR:
            tag = f"N{node_id}D{local_device_id}"
            tp = f"T{tp_rank}" if tp_rank is not None else ""
            it = f"_I{iteration_idx}" if iteration_idx is not None else ""
            self.logger = create_logger(
                "DCPExecutor",
                prefix=tag,
                log_file=f"executor/{tag}{tp}{it}.log",
            )
        self._instruction_handlers: Dict[type, Handler] = {}
        self.instr_index = 0
        self.return_values: Dict[int, Any] = {}
        self.buffers: Dict[str, Any] = {}
        self.buffer_n_blocks: Dict[str, int] = {}
        self.buffer_block_strides: Dict[str, int] = {}
        self.buffer_block_sizes: Dict[str, int] = {}
        self.buffer_per_token_shape: Dict[str, Tuple[int, ...]] = {}

    # -- ranks ---------------------------------------------------------------
    @property
    def rank(self):
        return self.get_rank(self.node_id, self.local_device_id)

    def get_rank(self, node_id: int, local_device_id: int):
        return node_id * self.n_devices_per_node + local_device_id

    def reverse_get_rank(self, rank: int):
        return divmod(rank, self.n_devices_per_node)

    # -- buffers -------------------------------------------------------------
    def init_forward_input(self, local_q, local_kv):
        self.buffers[BufferType.LOCAL_Q].copy_(local_q)
        self.buffers[BufferType.LOCAL_KV].copy_(local_kv)

    def init_backward_input(self, local_dout):
        self.buffers[BufferType.LOCAL_dOUT].copy_(local_dout)

    def deallocate_buffers(self):
        for buffer_type in self.buffers:
            if buffer_type in _TMP_BUFFER_TYPES:
                self.buffers[buffer_type] = None

    def init_buffers(self, execution_plan: ExecutionPlan):
        for buffer_type, info in execution_plan.buffer_info.items():
            self.buffer_n_blocks[buffer_type] = info.n_blocks
            self.buffer_block_strides[buffer_type] = info.block_numel
            self.buffer_block_sizes[buffer_type] = info.block_size
            self.buffer_per_token_shape[buffer_type] = info.per_token_shape
            if self.buffers.get(buffer_type) is None:
                if self.logger:
                    self.logger.debug(
                        "Creating buffer %s shape %s dtype %s per-token %s",
                        buffer_type,
                        info.buffer_shape,
                        info.dtype,
                        info.per_token_shape,
                    )
                self.buffers[buffer_type] = self._create_buffer(
                    info.buffer_shape, info.dtype
                )

    def _create_buffer(self, buffer_shape: Tuple[int, ...], buffer_dtype: int):
        raise NotImplementedError("DCPExecutor._create_buffer not implemented")

    # -- handler registry ----------------------------------------------------
    def register_handler(self, instruction_type, handler: Handler):
        if not (
            isinstance(instruction_type, type)
            and issubclass(instruction_type, BlockInstrBase)
        ):
            raise TypeError(
                "Instruction type must be a subclass of BlockInstrBase, got "
                f"{getattr(instruction_type, '__name__', instruction_type)}"
            )
        if instruction_type in self._instruction_handlers:
            raise ValueError(
                f"Instruction handler for {instruction_type.__name__} "
                "already registered."
            )
        self._instruction_handlers[instruction_type] = handler

    @classmethod
    def _get_leaf_subclasses(cls, instruction_type: Type[BlockInstrBase]):
        return _leaves(instruction_type)

    @classmethod
    def get_all_needed_handlers(cls):
        return sorted({t.__name__ for t in _leaves(BlockInstrBase)})

    def check_all_handlers_registered(self):
        for instruction_type in _leaves(BlockInstrBase):
            if instruction_type not in self._instruction_handlers:
                raise ValueError(
                    "No handler registered for instruction "
                    f"{instruction_type.__name__}"
                )

    def register_synchronization_handler(self, handler):
        self.synchronize = handler

    def synchronize(self):
        raise NotImplementedError("Synchronization handler not registered")

    # -- the loop ------------------------------------------------------------
    def execute(self, execution_plan: ExecutionPlan, is_forward: bool = True):
        self.execution_plan = execution_plan
        self.init_buffers(execution_plan)
        for index, instruction in enumerate(execution_plan.instructions):
            if self.logger:
                self.logger.debug("Executing instruction: %s", instruction)
            self.instr_index = index
            self._execute_instruction(instruction)
        if self.logger:
            self.logger.debug("Execution complete.")
        return self.return_values

    def _execute_instruction(self, instruction: BlockInstrBase):
        handler = self._instruction_handlers.get(type(instruction))
        if handler is None:
            raise ValueError(
                "No handler registered for instruction "
                f"{type(instruction).__name__}"
            )
        handler(self, instruction)
        if self.synchronous:
            self.synchronize()
