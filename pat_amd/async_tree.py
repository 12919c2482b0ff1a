"""`AsyncTree`: builds a decode step's tree, plan and device tensors on a helper thread.

Same constructor and `.tree` property as prefix_attn/async_tree.py:8-37 of the
flashserve/PAT tree: the vLLM backend creates one per decode step while earlier
work of the step is still running and blocks on `.tree` only when the first
attention layer needs the plan.
"""
from __future__ import annotations

import time
from concurrent.futures import Future, ThreadPoolExecutor
from typing import List, Optional, Union

import torch

from ._prefix_attn import PrefixTreeCPP

__all__ = ["AsyncTree"]

# one planner thread per process: plans of successive steps are built in order
_PLANNER = ThreadPoolExecutor(max_workers=1, thread_name_prefix="pat-plan")


_COPY_STREAMS: dict = {}


def _copy_stream(device: torch.device) -> "torch.cuda.Stream":
    """The planner thread's upload stream on `device` (default priority), created on first use."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    if index not in _COPY_STREAMS:
        _COPY_STREAMS[index] = torch.cuda.Stream(device=index)
    return _COPY_STREAMS[index]


class AsyncTree(PrefixTreeCPP):
    def __init__(self, block_size: int, seq_lens: Union[List[int], torch.Tensor], table: torch.Tensor,
                 MNWs: Optional[List[List[int]]], HRatio: int, kvHead: int, device: torch.device):
        super().__init__(block_size)
        self._tree: Optional[PrefixTreeCPP] = None
        self._init_time = time.time()

        def plan() -> PrefixTreeCPP:
            tree = PrefixTreeCPP(block_size)
            tree.build_radix_tree(seq_lens, table)
            tree.pack_schedule(MNWs=MNWs, HRatio=HRatio, kvHead=kvHead)
            dev = torch.device(device)
            if dev.type == "cuda":
                # the plan is one pinned buffer: its copy runs on a stream of its own, beside
                # whatever the model thread has queued, and is complete when this returns, so
                # the consumer may use any stream
                stream = _copy_stream(dev)
                with torch.cuda.stream(stream):
                    tree.kernel_info.to_gpu(dev)
                stream.synchronize()
            else:
                tree.kernel_info.to_gpu(dev)
            return tree

        self._future: Future = _PLANNER.submit(plan)

    @property
    def tree(self) -> PrefixTreeCPP:
        """The planned tree; waits for the helper thread and re-raises its exception."""
        if self._tree is None:
            self._tree = self._future.result()
            flat = self._tree.kernel_info._flat
            if flat is not None and flat.is_cuda:
                # allocated on the copy stream, read by kernels of the caller's stream
                flat.record_stream(torch.cuda.current_stream(flat.device))
        return self._tree
