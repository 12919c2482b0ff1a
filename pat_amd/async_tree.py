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
            tree.kernel_info.to_gpu(device)
            return tree

        self._future: Future = _PLANNER.submit(plan)

    @property
    def tree(self) -> PrefixTreeCPP:
        """The planned tree; waits for the helper thread and re-raises its exception."""
        if self._tree is None:
            self._tree = self._future.result()
        return self._tree
