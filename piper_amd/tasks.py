"""Task vocabulary of Piper's per-device executor, kept name-for-name (src/tasks.py:8-22) so that a
schedule written for the reference addresses the same tasks here.  Only the compute and update
tasks do work on one GPU; the communication tasks are accepted and are no-ops."""
from __future__ import annotations

from enum import Enum


class TaskType(Enum):
    FWD = "forward"
    BWD = "backward"
    UPD = "update"
    BWD_I = "backward_input"
    BWD_W = "backward_weight"
    FWD_BWD = "forward_backward"
    SEND = "send"
    RECV = "recv"
    ALL_REDUCE = "all_reduce"
    REDUCE_SCATTER = "reduce_scatter"
    ALL_GATHER = "all_gather"
    FWD_A2A = "forward_a2a"
    BWD_A2A = "backward_a2a"
    ORDER_DUMMY = "order_dummy"


COMPUTE_TASKS = frozenset({TaskType.FWD, TaskType.BWD, TaskType.BWD_I, TaskType.BWD_W, TaskType.FWD_BWD})
COMM_TASKS = frozenset({
    TaskType.SEND, TaskType.RECV, TaskType.ALL_REDUCE, TaskType.REDUCE_SCATTER,
    TaskType.ALL_GATHER, TaskType.FWD_A2A, TaskType.BWD_A2A,
})
