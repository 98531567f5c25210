"""End-to-end drop-in check of the attention backend: block manager + metadata builder +
MetaAttentionImpl.forward (append, prompt attention, chunked-prompt attention from the paged
cache, decode attention with eviction and block recycling) against an oracle simulation that
keeps every sequence's full K/V history in numpy.
Bit-exact: slot mapping, block tables, sequence lengths, every byte of every layer's KV tensor.
Within 2e-2 max-abs: attention outputs (bf16)."""
import numpy as np
import pytest
import torch

from oracle import attention as A
from oracle import paged as P

pytestmark = pytest.mark.gpu

HQ, HKV, D = 28, 4, 128
TOL = 2e-2


class OracleEngine:
    def __init__(self, layers, nb, bs, wl):
        self.model = P.WindowCacheModel(nb, bs, wl)
        self.wl, self.bs = wl, bs
        self.kc = [np.zeros((nb, bs, HKV, D), np.float32) for _ in range(layers)]
        self.vc = [np.zeros((nb, bs, HKV, D), np.float32) for _ in range(layers)]
        self.hist = {}                                       # seq -> per layer [(k rows), (v rows)]
        self.layers = layers

    def add(self, sid):
        self.model.add_seq(sid)
        self.hist[sid] = [[np.zeros((0, HKV, D), np.float32), np.zeros((0, HKV, D), np.float32)] for _ in range(self.layers)]

    def step(self, prompts, decodes, q, k, v, chunked=False):
        """q/k/v: per layer [T, H, D] float32 numpy, tokens laid out [prompts | decodes].
        Returns (slots, expected outputs per layer)."""
        slots, spans = [], []
        t = 0
        for sid, n in prompts:
            slots += self.model.append_tokens(sid, n, True, store_all=chunked); spans.append((sid, t, t + n)); t += n
        for d in decodes:
            sid, n = d if isinstance(d, tuple) else (d, 1)       # (sid, n): n query tokens for a decoding sequence
            slots += self.model.append_tokens(sid, n, False); spans.append((sid, t, t + n)); t += n
        outs = []
        for l in range(self.layers):
            P.kv_append(k[l], v[l], self.kc[l], self.vc[l], slots)
            out = np.zeros((t, HQ, D))
            for sid, a, b in spans:
                h = self.hist[sid][l]
                h[0] = np.concatenate([h[0], k[l][a:b]]); h[1] = np.concatenate([h[1], v[l][a:b]])
                out[a:b] = A.varlen_window_attention(q[l][a:b], h[0], h[1], [0, b - a], [0, len(h[0])], D ** -0.5, self.wl)
            outs.append(out)
        return slots, outs


def run_step(sb, dev, runner, impls, orc, prompts, decodes, g, chunked=False, dtype=torch.bfloat16):
    dec_tokens = sum(d[1] if isinstance(d, tuple) else 1 for d in decodes)
    T = sum(n for _, n in prompts) + dec_tokens
    layers = len(impls)
    q = [torch.randn(T, HQ, D, generator=g).to(dtype) for _ in range(layers)]
    k = [torch.randn(T, HKV, D, generator=g).to(dtype) for _ in range(layers)]
    v = [torch.randn(T, HKV, D, generator=g).to(dtype) for _ in range(layers)]
    meta = runner.build_step(prompts, decodes, chunked_prefill=chunked)
    slots, refs = orc.step(prompts, decodes, [x.float().numpy() for x in q], [x.float().numpy() for x in k],
                           [x.float().numpy() for x in v], chunked)
    assert meta.slot_mapping.cpu().tolist() == slots                                   # bit-exact indexing
    assert meta.num_prefill_tokens == sum(n for _, n in prompts) and meta.num_decode_tokens == dec_tokens
    if decodes:
        dm = meta.decode_metadata
        for i, d in enumerate(decodes):
            sid = d[0] if isinstance(d, tuple) else d
            table, seqlen, _ = orc.model.view(sid)
            assert dm.block_tables[i, :len(table)].cpu().tolist() == table
            assert (dm.block_tables[i, len(table):] == 0).all()
            assert int(dm.seq_lens_tensor[i]) == seqlen
    for l, impl in enumerate(impls):
        out = torch.full((T, HQ, D), float("nan"), dtype=dtype, device=dev)
        ret = impl.forward(None, q[l].to(dev), k[l].to(dev), v[l].to(dev), None, None, None, runner.kv_caches[l], meta, output=out)
        assert ret.data_ptr() == out.data_ptr()                                         # written in place
        err = np.abs(out.float().cpu().numpy() - refs[l]).max()
        assert err <= (TOL if dtype == torch.bfloat16 else 1e-5), f"layer {l}: max-abs {err}"
        assert np.array_equal(runner.kv_caches[l][0].float().cpu().numpy(), orc.kc[l])
        assert np.array_equal(runner.kv_caches[l][1].float().cpu().numpy(), orc.vc[l])
    return meta


@pytest.mark.parametrize("bs,wl", [(16, 64), (32, 80)])
def test_engine_prefill_decode_eviction(sb, dev, bs, wl):
    layers, nb = 2, 96
    g = torch.Generator().manual_seed(bs + wl)
    runner = sb.runner.SwaCacheRunner(layers, nb, bs, wl, HKV, D, torch.bfloat16, dev, max_seqs=4, max_chunk_tokens=256)
    impls = [sb.MetaAttentionImpl(HQ, D, D ** -0.5, HKV, None, wl + 1, "auto") for _ in range(layers)]
    orc = OracleEngine(layers, nb, bs, wl)
    for sid in (0, 1, 2):
        runner.add_seq(sid); orc.add(sid)
    # step 1: three prompts in one batch (shorter than, equal to and longer than the window)
    run_step(sb, dev, runner, impls, orc, [(0, 20), (1, wl), (2, 2 * wl + 5)], [], g)
    # steps 2..: all three decode; enough steps to cross several block boundaries (eviction + recycling)
    for _ in range(2 * bs + 3):
        run_step(sb, dev, runner, impls, orc, [], [0, 1, 2], g)
    # a new prompt arrives and is batched with the running decodes (prefill tokens first); mixed
    # batches only exist under chunked prefill, where the prompt attends through the paged cache
    runner.add_seq(3); orc.add(3)
    run_step(sb, dev, runner, impls, orc, [(3, 33)], [2, 0, 1], g, chunked=True)
    # sequence 1 finishes; its blocks go back to the stack and get reused by the others
    runner.free_seq(1); orc.model.free_seq(1)
    for _ in range(bs + 1):
        run_step(sb, dev, runner, impls, orc, [], [3, 0, 2], g)
    assert runner.manager.free_stack() == orc.model.free


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_engine_multi_query_decode(sb, dev, dtype):
    """Decoding sequences that take several query tokens in one step (max_decode_query_len > 1, the branch at
    vllm_hymeta/attention/meta_attention.py:924-953: varlen attention of the decode tokens over the paged
    cache): mixed run lengths in one batch, alone and behind a chunked prompt, across block boundaries and
    window eviction, interleaved with ordinary one-token steps. Slots, tables, lengths and cache bytes
    bit-exact; outputs against the oracle's varlen attention over each sequence's full history. bf16 takes
    the many-query kernel, fp32 one single-query row per token."""
    bs, wl, layers, nb = 16, 48, 2, 64
    g = torch.Generator().manual_seed(11)
    runner = sb.runner.SwaCacheRunner(layers, nb, bs, wl, HKV, D, dtype, dev, max_seqs=4, max_chunk_tokens=128)
    impls = [sb.MetaAttentionImpl(HQ, D, D ** -0.5, HKV, None, wl + 1, "auto") for _ in range(layers)]
    orc = OracleEngine(layers, nb, bs, wl)
    for sid in (0, 1, 2):
        runner.add_seq(sid); orc.add(sid)
    step = lambda prompts, decodes, chunked=False: run_step(sb, dev, runner, impls, orc, prompts, decodes, g,
                                                            chunked=chunked, dtype=dtype)
    step([(0, 10), (1, wl + 9), (2, 31)], [])
    meta = step([], [(0, 3), (1, 5), (2, 1)])                       # runs of 3, 5 and 1 query tokens
    assert meta.max_decode_query_len == 5 and meta.decode_metadata.query_start_loc.tolist() == [0, 3, 8, 9]
    step([], [0, 1, 2])                                             # an ordinary decode step in between
    for _ in range(6):                                              # 6 x 4 tokens: block boundaries, eviction, recycling
        step([], [(1, 4), (0, 4), (2, 2)])
    runner.add_seq(3); orc.add(3)
    step([(3, 40)], [(2, 3), (0, 2)], chunked=True)                 # behind a chunked prompt in the same batch
    step([], [(3, 17), (1, 2)])                                     # a run longer than a block
    assert runner.manager.free_stack() == orc.model.free


def test_engine_chunked_prefill_reads_paged_cache(sb, dev):
    bs, wl, layers, nb = 16, 64, 1, 64
    g = torch.Generator().manual_seed(5)
    runner = sb.runner.SwaCacheRunner(layers, nb, bs, wl, HKV, D, torch.bfloat16, dev, max_seqs=2, max_chunk_tokens=128)
    impls = [sb.MetaAttentionImpl(HQ, D, D ** -0.5, HKV, None, wl + 1, "auto")]
    orc = OracleEngine(layers, nb, bs, wl)
    for sid in (0, 1):
        runner.add_seq(sid); orc.add(sid)
    run_step(sb, dev, runner, impls, orc, [(0, 50), (1, 100)], [], g, chunked=True)      # first chunks
    run_step(sb, dev, runner, impls, orc, [(0, 70)], [1], g, chunked=True)               # second chunk + a decode
    run_step(sb, dev, runner, impls, orc, [(0, 30)], [1], g, chunked=True)
    for _ in range(20):
        run_step(sb, dev, runner, impls, orc, [], [0, 1], g)


def test_backend_static_interface(sb, dev):
    B = sb.MetaAttentionBackend
    assert B.get_name() == "META_FLASH_ATTN" and B.accept_output_buffer is True
    assert B.get_kv_cache_shape(10, 16, 4, 128) == (2, 10, 16, 4, 128)
    with pytest.raises(ValueError, match="multiple of 16"):
        B.get_kv_cache_shape(10, 8, 4, 128)
    assert B.get_impl_cls() is sb.MetaAttentionImpl and B.get_metadata_cls() is sb.MetaAttentionMetadata
    assert B.get_builder_cls() is sb.MetaAttentionMetadataBuilder
    assert B.get_supported_head_sizes() == [32, 64, 96, 128, 160, 192, 224, 256]   # the reference's list (meta_attention.py:57-59)
    # copy_blocks: copy-on-write inside each layer's cache, both halves
    g = torch.Generator().manual_seed(0)
    caches = [torch.randn(2, 6, 16, 4, 128, generator=g).bfloat16().to(dev) for _ in range(2)]
    before = [c.clone() for c in caches]
    pairs = torch.tensor([[0, 3], [1, 5], [0, 4]], dtype=torch.int64, device=dev)
    B.copy_blocks(caches, pairs)
    for c, b in zip(caches, before):
        exp = b.clone()
        for s, d in pairs.tolist():
            exp[:, d] = b[:, s]
        assert torch.equal(c, exp)
    # swap_blocks: device -> pinned host and back
    host = torch.zeros(2, 3, 16, 4, 128, dtype=torch.bfloat16, pin_memory=True)
    B.swap_blocks(caches[0], host, torch.tensor([[3, 0], [5, 2]]))
    torch.cuda.synchronize()
    assert torch.equal(host[:, 0], caches[0][:, 3].cpu()) and torch.equal(host[:, 2], caches[0][:, 5].cpu())
    fresh = torch.zeros_like(caches[0])
    B.swap_blocks(host, fresh, torch.tensor([[0, 1]]))
    torch.cuda.synchronize()
    assert torch.equal(fresh[:, 1].cpu(), host[:, 0])


def test_profile_run_and_errors(sb, dev):
    impl = sb.MetaAttentionImpl(HQ, D, D ** -0.5, HKV, None, 65, "auto")
    assert impl.sliding_window == (64, 0) and impl.num_queries_per_kv == 7
    assert sb.MetaAttentionImpl(HQ, D, 1.0, HKV, None, None, "auto").sliding_window == (-1, -1)
    # profiling run: empty kv_cache, prompt attention over the in-flight K/V, nothing appended
    T = 40
    g = torch.Generator().manual_seed(2)
    q = torch.randn(T, HQ, D, generator=g).bfloat16(); k = torch.randn(T, HKV, D, generator=g).bfloat16()
    v = torch.randn(T, HKV, D, generator=g).bfloat16()
    meta = sb.MetaAttentionMetadata(
        num_prefills=2, num_prefill_tokens=T, num_decode_tokens=0, slot_mapping=torch.full((T,), -1, dtype=torch.int64, device=dev),
        seq_lens=[15, 25], seq_lens_tensor=torch.tensor([15, 25], dtype=torch.int32, device=dev), max_prefill_seq_len=25,
        max_decode_seq_len=0, context_lens_tensor=torch.zeros(2, dtype=torch.int32, device=dev), block_tables=None,
        use_cuda_graph=False, max_query_len=25, max_decode_query_len=1,
        query_start_loc=torch.tensor([0, 15, 40], dtype=torch.int32, device=dev),
        seq_start_loc=torch.tensor([0, 15, 40], dtype=torch.int32, device=dev))
    out = torch.empty(T, HQ * D, dtype=torch.bfloat16, device=dev)                     # flat [T, Hq*D] is accepted
    impl.forward(None, q.to(dev).view(T, -1), k.to(dev).view(T, -1), v.to(dev).view(T, -1), None, None, None,
                 torch.empty(0, device=dev), meta, output=out)
    ref = A.varlen_window_attention(q.float().numpy(), k.float().numpy(), v.float().numpy(), [0, 15, 40], [0, 15, 40], D ** -0.5, 64)
    assert np.abs(out.view(T, HQ, D).float().cpu().numpy() - ref).max() <= TOL
    with pytest.raises(AssertionError, match="Output tensor"):
        impl.forward(None, q, k, v, None, None, None, torch.empty(0), meta, output=None)
    with pytest.raises(NotImplementedError, match="output quantization"):
        impl.forward(None, q, k, v, None, None, None, torch.empty(0), meta, output=out, output_scale=torch.ones(1))
    with pytest.raises(ValueError, match="blocksparse"):
        sb.MetaAttentionImpl(HQ, D, 1.0, HKV, None, 65, "auto", blocksparse_params={})
    for bad in (100, 16, 512):                             # sizes outside the list
        with pytest.raises(ValueError, match="Head size"):
            sb.MetaAttentionImpl(HQ, bad, 1.0, HKV, None, 65, "auto")
    with pytest.raises(NotImplementedError, match="KV sharing"):
        sb.MetaAttentionImpl(HQ, D, 1.0, HKV, None, 65, "auto", kv_sharing_target_layer_name="x")
    with pytest.raises(NotImplementedError, match="kv-cache"):
        sb.MetaAttentionImpl(HQ, D, 1.0, HKV, None, 65, "fp8_e5m2")
