"""vLLM v0 attention backend `PREFIX_ATTN` for ROCm: prefix-aware decode attention of libpat_amd
(MI355X) behind vLLM's backend interface.

Counterpart of plugin/vllm/attention/backends/prefix_attn.py of the flashserve/PAT tree
(backend :76-134, metadata :137-448, builder :451-686, impl :689-917), decoder-only models:
  * `PrefixAttentionBackend`          names the classes below and the cache layout
                                      `[2, num_blocks, block_size, kv_heads, head_size]`;
  * `PrefixAttentionMetadata`         a step's attention inputs; `decode_metadata` starts the
                                      step's plan (`pat_amd.vllm_decode.DecodePlan`: an AsyncTree on
                                      a helper thread) once and every layer reuses it;
                                      `advance_step` keeps the plan in step between the steps of
                                      multi-step decoding;
  * `PrefixAttentionMetadataBuilder`  per-request bookkeeping of a scheduler step: context lengths,
                                      block rows, slot mapping; for decode-only batches also the
                                      CPU copy of the padded block table and the head counts the
                                      planner needs (:609-619, :683-685);
  * `PrefixAttentionImpl.forward`     writes the step's K/V into the cache, runs prompt tokens
                                      through vLLM's flash attention and decode tokens through
                                      `prefix_attn_with_kvcache` (:901-915).
Encoder / cross attention, ALiBi, sliding windows, quantised caches and logit soft-capping are
refused, as in the reference (:718-737).

vLLM is imported when it is there; without it, small stand-ins for its base classes keep this
module importable so that the bookkeeping and the decode branch can be tested without vLLM.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from itertools import accumulate
from typing import Any, Dict, List, Optional, Tuple, Type

import torch

from pat_amd.utils import make_tensor_with_pad
from pat_amd.vllm_decode import DecodePlan, decode_attention

try:  # pragma: no cover - needs a vLLM checkout
    from vllm import _custom_ops as ops
    from vllm.attention.backends.abstract import (AttentionBackend, AttentionImpl, AttentionMetadata,
                                                  AttentionMetadataBuilder, AttentionType)
    from vllm.attention.backends.utils import (PAD_SLOT_ID, CommonAttentionState, compute_slot_mapping,
                                               compute_slot_mapping_start_idx, is_block_tables_empty)
    from vllm.utils import async_tensor_h2d
    HAVE_VLLM = True
except ImportError:
    HAVE_VLLM = False
    ops = None
    PAD_SLOT_ID = -1

    class AttentionBackend:  # stand-ins: just enough structure for the classes below
        pass

    class AttentionImpl:
        pass

    class AttentionMetadataBuilder:
        pass

    class CommonAttentionState:
        pass

    @dataclass
    class AttentionMetadata:
        num_prefills: int
        num_prefill_tokens: int
        num_decode_tokens: int
        slot_mapping: Optional[torch.Tensor]

    class AttentionType:
        DECODER = "decoder"

    def is_block_tables_empty(block_tables) -> bool:
        return block_tables is None or (isinstance(block_tables, dict) and all(v is None for v in block_tables.values()))

    def compute_slot_mapping_start_idx(is_prompt: bool, query_len: int, context_len: int, sliding_window) -> int:
        return 0    # (sliding windows are refused by this backend)

    def compute_slot_mapping(is_profile_run: bool, slot_mapping: List[int], seq_id: int, seq_len: int,
                             context_len: int, start_idx: int, block_size: int, block_tables) -> None:
        """Cache slot of every token of this step: block id * block_size + offset in the block."""
        if is_profile_run:
            slot_mapping.extend([PAD_SLOT_ID] * (seq_len - context_len))
            return
        row = block_tables[seq_id]
        for t in range(context_len, seq_len):
            slot_mapping.append(PAD_SLOT_ID if t < start_idx else row[t // block_size] * block_size + t % block_size)

    def async_tensor_h2d(data: list, dtype: torch.dtype, device, pin_memory: bool) -> torch.Tensor:
        t = torch.tensor(data, dtype=dtype, pin_memory=pin_memory and torch.cuda.is_available())
        return t.to(device=device, non_blocking=True)


def _flash_attn_varlen():
    """vLLM's ROCm flash attention for the prompt tokens (not part of this repository)."""
    try:  # pragma: no cover - needs a vLLM checkout
        from vllm.vllm_flash_attn import flash_attn_varlen_func
        return flash_attn_varlen_func
    except ImportError:
        try:  # pragma: no cover
            from flash_attn import flash_attn_varlen_func
            return flash_attn_varlen_func
        except ImportError as exc:
            raise NotImplementedError("prompt tokens need vLLM's flash attention (flash_attn_varlen_func); "
                                      "this backend only provides the decode path") from exc


class PrefixAttentionBackend(AttentionBackend):
    accept_output_buffer: bool = True

    @staticmethod
    def get_name() -> str:
        return "PREFIX_ATTN"

    @staticmethod
    def get_impl_cls() -> Type["PrefixAttentionImpl"]:
        return PrefixAttentionImpl

    @staticmethod
    def get_metadata_cls() -> Type["PrefixAttentionMetadata"]:
        return PrefixAttentionMetadata

    @staticmethod
    def get_builder_cls() -> Type["PrefixAttentionMetadataBuilder"]:
        return PrefixAttentionMetadataBuilder

    @staticmethod
    def get_state_cls():
        return CommonAttentionState

    @staticmethod
    def get_kv_cache_shape(num_blocks: int, block_size: int, num_kv_heads: int, head_size: int) -> Tuple[int, ...]:
        if block_size % 16 != 0:
            raise ValueError("Block size must be a multiple of 16.")
        return (2, num_blocks, block_size, num_kv_heads, head_size)

    @staticmethod
    def swap_blocks(src_kv_cache: torch.Tensor, dst_kv_cache: torch.Tensor, src_to_dst: torch.Tensor) -> None:
        for half in (0, 1):
            ops.swap_blocks(src_kv_cache[half], dst_kv_cache[half], src_to_dst)

    @staticmethod
    def copy_blocks(kv_caches: List[torch.Tensor], src_to_dists: torch.Tensor) -> None:
        ops.copy_blocks([c[0] for c in kv_caches], [c[1] for c in kv_caches], src_to_dists)


@dataclass
class PrefixAttentionMetadata(AttentionMetadata):
    """Rows are ordered prompts first, then decode requests (vLLM's batch layout)."""
    seq_lens: Optional[List[int]] = None
    seq_lens_tensor: Optional[torch.Tensor] = None
    max_query_len: Optional[int] = None
    max_decode_query_len: Optional[int] = 1
    max_prefill_seq_len: int = 0
    max_decode_seq_len: int = 0
    query_start_loc: Optional[torch.Tensor] = None
    seq_start_loc: Optional[torch.Tensor] = None
    context_lens_tensor: Optional[torch.Tensor] = None
    block_tables: Optional[torch.Tensor] = None
    use_cuda_graph: bool = False
    block_size: int = 16
    # what the planner needs, kept for decode-only steps (the reference's builder, :609-619, :683-685)
    block_tables_cpu: Optional[torch.Tensor] = None
    nheads: Optional[int] = None
    nheads_kv: Optional[int] = None
    multi_modal_placeholder_index_maps: Optional[Dict[str, Any]] = None
    enable_kv_scales_calculation: bool = True
    _cached_prefill_metadata: Optional["PrefixAttentionMetadata"] = field(default=None, repr=False)
    _cached_decode_plan: Optional[DecodePlan] = field(default=None, repr=False)

    @property
    def prefill_metadata(self) -> Optional["PrefixAttentionMetadata"]:
        if self.num_prefills == 0:
            return None
        if self._cached_prefill_metadata is None:
            n, t = self.num_prefills, self.num_prefill_tokens
            cut = lambda x, k: None if x is None else x[:k]
            self._cached_prefill_metadata = PrefixAttentionMetadata(
                num_prefills=n, num_prefill_tokens=t, num_decode_tokens=0, slot_mapping=cut(self.slot_mapping, t),
                seq_lens=cut(self.seq_lens, n), seq_lens_tensor=cut(self.seq_lens_tensor, n),
                max_query_len=self.max_query_len, max_decode_query_len=0, max_prefill_seq_len=self.max_prefill_seq_len,
                max_decode_seq_len=0, query_start_loc=cut(self.query_start_loc, n + 1),
                seq_start_loc=cut(self.seq_start_loc, n + 1), context_lens_tensor=cut(self.context_lens_tensor, n),
                block_tables=cut(self.block_tables, n), use_cuda_graph=False, block_size=self.block_size,
                multi_modal_placeholder_index_maps=self.multi_modal_placeholder_index_maps,
                enable_kv_scales_calculation=self.enable_kv_scales_calculation)
        return self._cached_prefill_metadata

    @property
    def decode_metadata(self) -> Optional[DecodePlan]:
        """The decode side of the step: its requests' lengths and block rows and the plan, whose
        construction starts here on the helper thread the first time a layer asks (:313-338)."""
        if self.num_decode_tokens == 0:
            return None
        if self._cached_decode_plan is None:
            assert self.block_tables_cpu is not None and self.nheads and self.nheads_kv, \
                "PREFIX_ATTN plans decode-only steps: the builder keeps block_tables_cpu / nheads / nheads_kv for those"
            self._cached_decode_plan = DecodePlan.from_metadata(self)
        return self._cached_decode_plan

    def advance_step(self, block_tables_cpu: torch.Tensor, num_seqs: int, num_queries: int) -> None:
        """Between the steps of multi-step decoding: every request has one more token. The
        reference moves the lengths forward and leaves the plan as it was (:377-448); here the plan
        grows with them, in place where it can."""
        assert self.num_prefills == 0 and self.num_prefill_tokens == 0 and self.num_decode_tokens == num_seqs
        assert num_seqs == num_queries and self.seq_lens is not None and len(self.seq_lens) == num_seqs
        for i in range(num_queries):
            self.seq_lens[i] += 1
        self.max_decode_seq_len = max(self.seq_lens)
        if self.seq_lens_tensor is not None:
            self.seq_lens_tensor[:num_queries] += 1
        self.block_tables_cpu = block_tables_cpu
        if self._cached_decode_plan is not None:
            self._cached_decode_plan.advance_step(block_tables_cpu)


class PrefixAttentionMetadataBuilder(AttentionMetadataBuilder):
    def __init__(self, input_builder: Any):
        self.input_builder = input_builder
        self.runner = input_builder.runner
        self.sliding_window = input_builder.sliding_window
        self.block_size = input_builder.block_size

    def prepare(self) -> None:
        self.slot_mapping: List[int] = []
        self.prefill_seq_lens: List[int] = []
        self.context_lens: List[int] = []
        self.block_tables: List[List[int]] = []
        self.curr_seq_lens: List[int] = []
        self.num_prefills = 0
        self.num_prefill_tokens = 0
        self.num_decode_tokens = 0

    def _add_seq_group(self, inter_data: Any, chunked_prefill_enabled: bool, prefix_cache_hit: bool) -> None:
        """One scheduled group: counts its tokens on the prompt or the decode side, records its
        requests' block rows and the cache slots its new tokens are written to."""
        tables = inter_data.block_tables
        profile_run = is_block_tables_empty(tables)
        for i, seq_id in enumerate(inter_data.seq_ids):
            query_len, context_len = inter_data.query_lens[i], inter_data.context_lens[i]
            self.context_lens.append(context_len)
            if inter_data.is_prompt:
                self.num_prefills += 1
                self.num_prefill_tokens += len(inter_data.input_tokens[i])
                self.prefill_seq_lens.append(inter_data.orig_seq_lens[i])
            else:
                self.num_decode_tokens += query_len
                self.curr_seq_lens.append(inter_data.seq_lens[i])
            row: List[int] = []
            if tables is not None and (prefix_cache_hit or chunked_prefill_enabled or not inter_data.is_prompt):
                window = 0 if prefix_cache_hit else inter_data.curr_sliding_window_blocks[i]
                row = tables[seq_id] if window == 0 else tables[seq_id][-window:]
            self.block_tables.append(row)
            start = compute_slot_mapping_start_idx(inter_data.is_prompt, query_len, context_len, self.sliding_window)
            compute_slot_mapping(profile_run, self.slot_mapping, seq_id, inter_data.orig_seq_lens[i], context_len,
                                 start, self.block_size, tables)

    def build(self, seq_lens: List[int], query_lens: List[int], cuda_graph_pad_size: int,
              batch_size: int) -> PrefixAttentionMetadata:
        """Device tensors of the step. `cuda_graph_pad_size` is -1 when the step is not replayed from a
        captured graph; the plan of a decode step is data dependent, so graph replay of decode steps is
        not offered here (the reference marks its metadata `use_cuda_graph=False` too, :300)."""
        if cuda_graph_pad_size != -1:
            raise NotImplementedError("PREFIX_ATTN plans every decode step afresh: run with enforce_eager")
        hit = any(d.prefix_cache_hit for d in self.input_builder.inter_data_list)
        for d in self.input_builder.inter_data_list:
            self._add_seq_group(d, self.input_builder.chunked_prefill_enabled, hit)
        device = self.runner.device
        pin = getattr(self.runner, "pin_memory", False)
        decode_query_lens = query_lens[self.num_prefills:]
        table_cpu = nheads = nheads_kv = None
        if self.num_prefills == 0:
            # a decode-only step: the planner reads the padded table on the host (helper thread) while
            # its copy travels to the device
            table_cpu = make_tensor_with_pad(self.block_tables, pad=0, dtype=torch.int, device="cpu")
            tables = table_cpu.to(device=device, non_blocking=True)
            nheads = self.runner.model_config.get_num_attention_heads(self.runner.parallel_config)
            nheads_kv = self.runner.model_config.get_num_kv_heads(self.runner.parallel_config)
            assert nheads and nheads_kv, "head counts must be known to plan the decode step"
        else:
            tables = make_tensor_with_pad(self.block_tables, pad=0, dtype=torch.int, device=device)
        h2d = lambda data, dtype: async_tensor_h2d(data, dtype, device, pin)
        return PrefixAttentionMetadata(
            num_prefills=self.num_prefills, num_prefill_tokens=self.num_prefill_tokens,
            num_decode_tokens=self.num_decode_tokens, slot_mapping=h2d(self.slot_mapping, torch.long),
            seq_lens=seq_lens, seq_lens_tensor=h2d(seq_lens, torch.int), max_query_len=max(query_lens),
            max_decode_query_len=max(decode_query_lens, default=1),
            max_prefill_seq_len=max(self.prefill_seq_lens, default=0),
            max_decode_seq_len=max(self.curr_seq_lens, default=0),
            query_start_loc=h2d(list(accumulate(query_lens, initial=0)), torch.int32),
            seq_start_loc=h2d(list(accumulate(seq_lens, initial=0)), torch.int32),
            context_lens_tensor=h2d(self.context_lens, torch.int), block_tables=tables, use_cuda_graph=False,
            block_size=self.block_size, block_tables_cpu=table_cpu, nheads=nheads, nheads_kv=nheads_kv)


def _write_kv_cache(key: torch.Tensor, value: torch.Tensor, kv_cache: torch.Tensor, slots: torch.Tensor,
                    kv_cache_dtype: str, layer: Any) -> None:
    """The step's new K/V rows go to their cache slots: vLLM's reshape_and_cache_flash (:828-837)
    when vLLM is there; without it, the same scatter with torch (tests only)."""
    if HAVE_VLLM:  # pragma: no cover
        torch.ops._C_cache_ops.reshape_and_cache_flash(key, value, kv_cache[0], kv_cache[1], slots, kv_cache_dtype,
                                                        layer._k_scale, layer._v_scale)
        return
    live = slots >= 0
    flat_k = kv_cache[0].view(-1, *kv_cache.shape[3:])
    flat_v = kv_cache[1].view(-1, *kv_cache.shape[3:])
    flat_k.index_copy_(0, slots[live], key[:slots.numel()][live])
    flat_v.index_copy_(0, slots[live], value[:slots.numel()][live])


class PrefixAttentionImpl(AttentionImpl):
    """query / output: [num_tokens, num_heads, head_size], prompt tokens first, then one token per
    decode request; kv_cache: [2, num_blocks, block_size, num_kv_heads, head_size]."""

    def __init__(self, num_heads: int, head_size: int, scale: float, num_kv_heads: int,
                 alibi_slopes: Optional[List[float]] = None, sliding_window: Optional[int] = None,
                 kv_cache_dtype: str = "auto", blocksparse_params: Optional[Dict[str, Any]] = None,
                 logits_soft_cap: Optional[float] = None, attn_type: str = AttentionType.DECODER,
                 use_irope: bool = False) -> None:
        if blocksparse_params is not None:
            raise ValueError("PrefixAttention does not support block-sparse attention.")
        for what, given in (("alibi slopes", alibi_slopes), ("sliding window", sliding_window),
                            ("logits soft cap", logits_soft_cap)):
            if given is not None:
                raise NotImplementedError(f"PrefixAttention does not support {what} currently.")
        if kv_cache_dtype not in ("auto", "float16", "bfloat16", "half"):
            raise NotImplementedError(f"PrefixAttention does not support {kv_cache_dtype} kv-cache currently.")
        if attn_type != AttentionType.DECODER:
            raise NotImplementedError("PrefixAttention serves decoder self-attention only.")
        assert num_heads % num_kv_heads == 0
        self.num_heads, self.head_size, self.scale, self.num_kv_heads = num_heads, head_size, float(scale), num_kv_heads
        self.num_queries_per_kv = num_heads // num_kv_heads
        self.kv_cache_dtype = kv_cache_dtype
        self.attn_type = attn_type

    def forward(self, layer: Any, query: torch.Tensor, key: Optional[torch.Tensor], value: Optional[torch.Tensor],
                kv_cache: torch.Tensor, attn_metadata: PrefixAttentionMetadata,
                output: Optional[torch.Tensor] = None) -> torch.Tensor:
        assert output is not None, "Output tensor must be provided."
        assert getattr(layer, "_k_scale_float", 1.0) == 1.0 and getattr(layer, "_v_scale_float", 1.0) == 1.0, \
            "PrefixAttention supports only kv_cache type of FP16 and BF16"
        if kv_cache.numel() > 0 and key is not None and value is not None:
            _write_kv_cache(key, value, kv_cache, attn_metadata.slot_mapping.flatten(), self.kv_cache_dtype, layer)
        n_prefill = attn_metadata.num_prefill_tokens
        n_decode = attn_metadata.num_decode_tokens
        assert query.shape[0] >= n_prefill + n_decode

        prefill = attn_metadata.prefill_metadata
        if prefill is not None:
            flash = _flash_attn_varlen()
            fresh = kv_cache.numel() == 0 or prefill.block_tables is None or prefill.block_tables.numel() == 0
            if fresh:       # prompts with nothing cached: attention over the step's own K/V
                flash(q=query[:n_prefill], k=key[:n_prefill], v=value[:n_prefill], cu_seqlens_q=prefill.seq_start_loc,
                      cu_seqlens_k=prefill.seq_start_loc, max_seqlen_q=prefill.max_prefill_seq_len,
                      max_seqlen_k=prefill.max_prefill_seq_len, softmax_scale=self.scale, causal=True,
                      out=output[:n_prefill])
            else:           # prefix-cache hit or chunked prefill: keys come from the paged cache
                flash(q=query[:n_prefill], k=kv_cache[0], v=kv_cache[1], cu_seqlens_q=prefill.query_start_loc,
                      max_seqlen_q=prefill.max_query_len, seqused_k=prefill.seq_lens_tensor,
                      max_seqlen_k=max(prefill.seq_lens), softmax_scale=self.scale, causal=True,
                      block_table=prefill.block_tables, out=output[:n_prefill])

        plan = attn_metadata.decode_metadata
        if plan is not None:
            decode_attention(query[n_prefill:n_prefill + n_decode], kv_cache, plan, self.scale,
                             output[n_prefill:n_prefill + n_decode])
        return output
