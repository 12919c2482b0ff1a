"""The ROCm overlay of the vLLM `PREFIX_ATTN` backend (plugin/vllm_rocm) without vLLM: the metadata
builder's bookkeeping against a stand-in for vLLM's model-input builder, the metadata's decode
side, and `PrefixAttentionImpl.forward` on a decode-only step on the GPU."""
import math
from types import SimpleNamespace

import pytest
import torch

from oracle import attn_oracle as ao
from pat_amd import PrefixTree, workloads
from plugin.vllm_rocm.attention.backends import prefix_attn as backend
from conftest import plan_fields


def _decode_group(seq_id, row, seq_len):
    """What vLLM's input builder holds for one running request that decodes one token."""
    return SimpleNamespace(is_prompt=False, seq_ids=[seq_id], block_tables={seq_id: list(row)}, input_tokens=[[1]],
                           orig_seq_lens=[seq_len], seq_lens=[seq_len], query_lens=[1], context_lens=[seq_len - 1],
                           curr_sliding_window_blocks=[0], prefix_cache_hit=False)


def _prompt_group(seq_id, row, n_tokens):
    return SimpleNamespace(is_prompt=True, seq_ids=[seq_id], block_tables={seq_id: list(row)},
                           input_tokens=[list(range(n_tokens))], orig_seq_lens=[n_tokens], seq_lens=[n_tokens],
                           query_lens=[n_tokens], context_lens=[0], curr_sliding_window_blocks=[0],
                           prefix_cache_hit=False)


def _input_builder(groups, w, device):
    config = SimpleNamespace(get_num_attention_heads=lambda pc: w.heads, get_num_kv_heads=lambda pc: w.kv_heads)
    runner = SimpleNamespace(device=device, pin_memory=False, model_config=config, parallel_config=None)
    return SimpleNamespace(runner=runner, sliding_window=None, block_size=w.page_size, inter_data_list=groups,
                           chunked_prefill_enabled=False)


def _build_decode_step(w, device):
    groups = [_decode_group(100 + i, w.rows[i], w.seq_lens[i]) for i in range(w.batch)]
    b = backend.PrefixAttentionMetadataBuilder(_input_builder(groups, w, device))
    b.prepare()
    return b.build(list(w.seq_lens), [1] * w.batch, -1, w.batch)


def test_backend_names_its_parts():
    be = backend.PrefixAttentionBackend
    assert be.get_name() == "PREFIX_ATTN" and be.accept_output_buffer
    assert be.get_impl_cls() is backend.PrefixAttentionImpl
    assert be.get_metadata_cls() is backend.PrefixAttentionMetadata
    assert be.get_builder_cls() is backend.PrefixAttentionMetadataBuilder
    assert be.get_kv_cache_shape(7, 32, 8, 128) == (2, 7, 32, 8, 128)
    with pytest.raises(ValueError, match="multiple of 16"):
        be.get_kv_cache_shape(7, 8, 8, 128)


def test_builder_bookkeeping_of_a_decode_only_step():
    w = workloads.make("c1", seed=5)
    meta = _build_decode_step(w, torch.device("cpu"))
    assert (meta.num_prefills, meta.num_prefill_tokens, meta.num_decode_tokens) == (0, 0, w.batch)
    assert meta.seq_lens == list(w.seq_lens) and meta.max_decode_seq_len == max(w.seq_lens)
    assert meta.max_query_len == 1 and meta.max_decode_query_len == 1 and meta.max_prefill_seq_len == 0
    assert meta.context_lens_tensor.tolist() == [n - 1 for n in w.seq_lens]
    assert meta.query_start_loc.tolist() == list(range(w.batch + 1))
    assert meta.seq_start_loc.tolist()[-1] == sum(w.seq_lens)
    # the planner's inputs: the padded table on the host, its device copy, the head counts
    assert torch.equal(meta.block_tables_cpu, w.padded_table()) and torch.equal(meta.block_tables, w.padded_table())
    assert (meta.nheads, meta.nheads_kv, meta.block_size) == (w.heads, w.kv_heads, w.page_size)
    # every request writes its new token (position seq_len - 1) to that token's cache slot
    want = [w.rows[i][(n - 1) // w.page_size] * w.page_size + (n - 1) % w.page_size for i, n in enumerate(w.seq_lens)]
    assert meta.slot_mapping.tolist() == want
    assert meta.prefill_metadata is None


def test_builder_keeps_no_planner_inputs_for_steps_with_prompts():
    w = workloads.make("c1", seed=5)
    groups = [_prompt_group(7, [40, 41], 20)] + [_decode_group(100 + i, w.rows[i], w.seq_lens[i]) for i in range(2)]
    b = backend.PrefixAttentionMetadataBuilder(_input_builder(groups, w, torch.device("cpu")))
    b.prepare()
    meta = b.build([20] + list(w.seq_lens[:2]), [20, 1, 1], -1, 22)
    assert (meta.num_prefills, meta.num_prefill_tokens, meta.num_decode_tokens) == (1, 20, 2)
    assert meta.block_tables_cpu is None and meta.nheads is None
    assert meta.max_prefill_seq_len == 20 and meta.max_query_len == 20
    assert meta.slot_mapping.tolist()[:20] == [40 * 16 + t for t in range(16)] + [41 * 16 + t for t in range(4)]
    assert meta.block_tables[0].tolist()[:2] == [0, 0]       # a prompt without cache hit carries no block row
    pre = meta.prefill_metadata
    assert pre.num_prefills == 1 and pre.num_decode_tokens == 0 and pre.seq_lens == [20]
    assert pre.slot_mapping.numel() == 20 and pre.query_start_loc.tolist() == [0, 20]
    with pytest.raises(NotImplementedError, match="enforce_eager"):
        b.prepare()
        b.build([20], [20], 3, 8)


def test_decode_metadata_plans_once_and_advances():
    w = workloads.make("c1", seed=5)
    meta = _build_decode_step(w, torch.device("cpu"))
    plan = meta.decode_metadata
    assert plan is meta.decode_metadata                           # every layer of the step gets the same plan
    ref = PrefixTree(w.page_size)
    ref.build_radix_tree(w.seq_lens, w.rows)
    want = plan_fields(ref.pack_schedule(MNWs=None, HRatio=w.heads // w.kv_heads, kvHead=w.kv_heads))
    got = plan.tree.tree.kernel_info
    assert [list(m) for m in got.MNWs] == want["MNWs"]
    assert [t.tolist() for t in got.kv_in_CTAs] == want["kv_in_CTAs"]
    # multi-step decoding: one more token per request (same blocks: 288 -> 289 tokens need a 19th block)
    table = torch.zeros(w.batch, w.padded_table().shape[1] + 1, dtype=torch.int32)
    table[:, :-1] = w.padded_table()
    table[:, -1] = torch.arange(900, 900 + w.batch, dtype=torch.int32)
    meta.advance_step(table, w.batch, w.batch)
    assert meta.seq_lens == [n + 1 for n in w.seq_lens] and plan.seq_lens == meta.seq_lens
    assert meta.max_decode_seq_len == max(w.seq_lens) + 1


def test_impl_refuses_what_the_kernels_do_not_do():
    mk = lambda **kw: backend.PrefixAttentionImpl(8, 64, 0.125, 8, **kw)
    with pytest.raises(NotImplementedError, match="alibi"):
        mk(alibi_slopes=[1.0])
    with pytest.raises(NotImplementedError, match="sliding window"):
        mk(sliding_window=128)
    with pytest.raises(NotImplementedError, match="fp8"):
        mk(kv_cache_dtype="fp8")
    with pytest.raises(ValueError, match="block-sparse"):
        mk(blocksparse_params={})
    assert mk().num_queries_per_kv == 1


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["c1", "c2"])
def test_impl_forward_decode_only_step(name):
    # one decode step as vLLM drives it: the step's K/V rows are written to their cache slots, then
    # every request attends to its whole context through the plan
    print(f"[case] PrefixAttentionImpl.forward, decode-only step, {name}", flush=True)
    dev = torch.device("cuda:0")
    w = workloads.make(name, seed=6)
    q, k, v = w.tensors(dev)
    meta = _build_decode_step(w, dev)
    slots = meta.slot_mapping
    flat_k, flat_v = k.view(-1, w.kv_heads, w.head_dim), v.view(-1, w.kv_heads, w.head_dim)
    new_k, new_v = flat_k[slots].clone(), flat_v[slots].clone()
    kv_cache = torch.stack([k, v])
    kv_cache[0].view(-1, w.kv_heads, w.head_dim)[slots] = 0       # the cache before the step: last tokens missing
    kv_cache[1].view(-1, w.kv_heads, w.head_dim)[slots] = 0
    impl = backend.PrefixAttentionImpl(w.heads, w.head_dim, 1.0 / math.sqrt(w.head_dim), w.kv_heads)
    query = q.squeeze(1).contiguous()
    output = torch.full_like(query, float("nan"))
    layer = SimpleNamespace(_k_scale_float=1.0, _v_scale_float=1.0, _k_scale=None, _v_scale=None)
    for _ in range(2):                                            # two layers of the step share the plan
        impl.forward(layer, query, new_k, new_v, kv_cache, meta, output)
    torch.cuda.synchronize()
    assert torch.equal(kv_cache[0], k) and torch.equal(kv_cache[1], v)
    ref, _ = ao.paged_attention_ref(q.cpu(), k.cpu(), v.cpu(), w.rows, w.seq_lens)
    err = (output.unsqueeze(1).float().cpu() - ref.float()).abs().max().item()
    tol = 2e-3 if w.dtype == torch.float16 else 1.6e-2
    print(f"[parity] backend forward {name}: max|out - ref| = {err:.3e} (tol {tol:.1e})", flush=True)
    assert err <= tol
