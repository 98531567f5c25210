"""Host-side logic that needs no GPU: the metadata builder driven by the runner slice, the
prefill/decode views of the metadata, and the GLA slot cache bookkeeping."""
import numpy as np
import pytest
import torch

from oracle import paged as P


def test_builder_matches_model_on_cpu_tensors(sb):
    bs, wl, nb = 16, 48, 64
    runner = sb.SwaCacheRunner(1, nb, bs, wl, 2, 128, torch.float32, "cpu", max_seqs=3, max_chunk_tokens=200)
    model = P.WindowCacheModel(nb, bs, wl)
    for s in (7, 8, 9):
        runner.add_seq(s); model.add_seq(s)
    meta = runner.build_step([(7, 10), (8, 130)], [])
    exp = model.append_tokens(7, 10, True) + model.append_tokens(8, 130, True)
    assert meta.slot_mapping.tolist() == exp and meta.slot_mapping.dtype == torch.int64
    assert meta.num_prefills == 2 and meta.num_prefill_tokens == 140 and meta.num_decode_tokens == 0
    assert meta.seq_lens == [10, 130] and meta.max_prefill_seq_len == 130 and meta.max_query_len == 130
    assert meta.query_start_loc.tolist() == [0, 10, 140] and meta.seq_start_loc.tolist() == [0, 10, 140]
    assert meta.block_tables.numel() == 0                     # plain prompts attend over the in-flight K/V
    assert meta.context_lens_tensor.tolist() == [0, 0]
    assert meta.decode_metadata is None and meta.prefill_metadata.num_prefill_tokens == 140

    meta = runner.build_step([(9, 20)], [8, 7])               # mixed step: prefill tokens first
    exp = model.append_tokens(9, 20, True) + model.append_tokens(8, 1, False) + model.append_tokens(7, 1, False)
    assert meta.slot_mapping.tolist() == exp
    pm, dm = meta.prefill_metadata, meta.decode_metadata
    assert pm.slot_mapping.tolist() == exp[:20] and dm.slot_mapping.tolist() == exp[20:]
    assert dm.query_start_loc.tolist() == [0, 1, 2] and pm.query_start_loc.tolist() == [0, 20]
    assert dm.num_decode_tokens == 2 and dm.max_decode_query_len == 1
    for i, s in enumerate((8, 7)):
        table, seqlen, _ = model.view(s)
        assert dm.block_tables[i, :len(table)].tolist() == table and dm.block_tables.dtype == torch.int32
        assert int(dm.seq_lens_tensor[i]) == seqlen
    assert dm.max_decode_seq_len == max(model.view(8)[1], model.view(7)[1])
    assert meta.prefill_metadata is pm and meta.decode_metadata is dm   # views are cached

    for _ in range(3 * bs):                                   # window slides, tables stay window-bounded
        meta = runner.build_step([], [7, 8, 9])
        exp = [model.append_tokens(s, 1, False)[0] for s in (7, 8, 9)]
        assert meta.slot_mapping.tolist() == exp
        assert meta.block_tables.shape[1] <= wl // bs + 2
        for i, s in enumerate((7, 8, 9)):
            table, seqlen, _ = model.view(s)
            assert meta.block_tables[i, :len(table)].tolist() == table and int(meta.seq_lens_tensor[i]) == seqlen


def test_builder_graph_padding(sb):
    bs, wl = 16, 32
    runner = sb.SwaCacheRunner(1, 16, bs, wl, 2, 128, torch.float32, "cpu", max_seqs=2)
    runner.add_seq(0)
    runner.build_step([(0, 5)], [])
    mgr = runner.manager
    from spikingbrain_7b_amd.runner import ResidentTable, SeqGroupData, _InputBuilder, _Runner
    mgr.decode_step([0])
    r = mgr.row_of(0)
    rn = _Runner(torch.device("cpu"), graph_block_tables=np.zeros((4, 8), np.int32))
    ib = _InputBuilder(rn, wl, bs, False)
    ib.inter_data_list.append(SeqGroupData(False, [0], [[0]], [6], [6], [1], [5], [1], {0: ResidentTable(mgr, r)}))
    b = sb.MetaAttentionMetadataBuilder(ib)
    b.prepare()
    meta = b.build([6, 1, 1, 1], [1, 1, 1, 1], cuda_graph_pad_size=3, batch_size=4)
    assert meta.use_cuda_graph and meta.num_decode_tokens == 4
    assert meta.slot_mapping.tolist()[1:] == [sb.PAD_SLOT_ID] * 3       # padded lanes never write
    assert meta.block_tables.shape == (4, 8) and meta.block_tables[1:].abs().sum() == 0


def test_gla_slot_cache_bookkeeping(sb):
    m = sb.GLACacheManager(torch.float32, (2, 4, 1, 8, 8), device="cpu")
    m.cache.copy_(torch.arange(2 * 4 * 64, dtype=torch.float32).view(2, 4, 1, 8, 8))
    cache, idx = m.current_run_tensors(request_ids_to_seq_ids={"a": [0], "b": [1]}, finished_requests_ids=[])
    assert idx.tolist() == [3, 2] and idx.dtype == torch.int32 and cache is m.cache      # highest free slot first
    # parallel sampling: a new sequence of a known request gets a copy of its sibling's state
    _, idx = m.current_run_tensors(request_ids_to_seq_ids={"a": [0, 5], "b": [1]}, finished_requests_ids=[])
    assert idx.tolist() == [3, 1, 2]
    assert torch.equal(m.cache[:, 1], m.cache[:, 3])
    # finished request: slots go back, and the id maps to PAD in the same step
    _, idx = m.current_run_tensors(request_ids_to_seq_ids={"a": [0, 5], "c": [9]}, finished_requests_ids=["b"])
    assert idx.tolist() == [3, 1, 2]                                                       # c reuses b's slot 2
    _, idx = m.current_run_tensors(request_ids_to_seq_ids={"a": [0]}, finished_requests_ids=["a"])
    assert idx.tolist() == [sb.PAD_SLOT_ID]
    # per-layer view
    p = sb.GLACacheParams(m.cache, idx).at_layer_idx(1)
    assert p.gla_cache.shape == (4, 1, 8, 8) and p.gla_cache.data_ptr() == m.cache[1].data_ptr()
    # brand-new prompts (context 0) get their slot zeroed in every layer, running ones do not
    from spikingbrain_7b_amd.gla import clear_prefill_slots
    m2 = sb.GLACacheManager(torch.float32, (2, 3, 1, 8, 8), device="cpu")
    m2.cache.fill_(float("nan"))
    m2.current_run_tensors(request_ids_to_seq_ids={"x": [10], "y": [11]}, finished_requests_ids=[])
    cleared = clear_prefill_slots(m2, 2, [0, 17], {"x": [10], "y": [11]})
    assert cleared == [2] and (m2.cache[:, 2] == 0).all() and m2.cache[:, 1].isnan().all()
    cap = m2.get_seqlen_agnostic_capture_inputs(5)
    assert cap[1].tolist() == [sb.PAD_SLOT_ID] * 5


def test_cache_is_a_transformers_cache(sb):
    """hf_7B_model/cache.py:11 derives from transformers.cache_utils.Cache: code that checks the type (HF
    generate plumbing) must accept the drop-in, and the container protocol must be the class's own."""
    from transformers.cache_utils import Cache as HFCache
    c = sb.Cache(seen_tokens=3)
    assert isinstance(c, HFCache)
    assert len(c) == 0 and list(c) == [] and c.get_seq_length(0) == 0 and c.get_max_length() is None
    assert c._seen_tokens == 3
    with pytest.raises(KeyError):
        c[0]
    legacy = ({"recurrent_state": None, "attn_state": None, "conv_state": None},)
    c2 = sb.Cache.from_legacy_cache(legacy, seen_tokens=7)
    assert isinstance(c2, HFCache) and len(c2) == 1 and c2.get_seq_length(0) == 7 and c2.to_legacy_cache() == legacy
