"""Writes tests/golden/cache_path_v1.npz: small input/expected-output vectors for every part of the
cache path, computed by the CPU oracle (oracle/) at the time the oracle was pinned by its own tests.

The reference ships no golden vectors for this path and none of its modules was imported to make
these: they are a regression pin. If the oracle (or a kernel) later drifts, tests/test_golden.py
fails against data that does not move with the code. Inputs are stored explicitly (bf16 tensors as
their uint16 bit patterns), so nothing depends on a random-number generator at test time.

cache_path_v2_ext.npz holds the same kind of vectors for the paths added later (per-row INT8 K/V,
meta-token attention, GLA over a prompt, a ragged decode batch); it is a file of its own so that v1
never changes.

    python tests/golden/make_fixtures.py        # rewrites both .npz files (deterministic)
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import attention as A  # noqa: E402
from oracle import gla as G  # noqa: E402
from oracle import paged as P  # noqa: E402
from oracle.hf_cache import OracleCache  # noqa: E402


def bf16_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> bf16 bit patterns, round to nearest even."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF).astype(np.uint16)


def bf16_to_f32(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << 16).view(np.float32)


def main() -> None:
    rng = np.random.default_rng(20240607)
    out = {}

    # 1. dense HF cache: window 8, ragged appends incl. first-call truncation, cat, == W roll, overshoot
    W, H, D = 8, 2, 4
    steps = [11, 1, 1, 3, 1, 2, 1]
    cache = OracleCache()
    stream_k = rng.integers(-50, 50, size=(1, H, sum(steps), D)).astype(np.float32)
    stream_v = rng.integers(-50, 50, size=(1, H, sum(steps), D)).astype(np.float32)
    t = 0
    for i, n in enumerate(steps):
        k, v = stream_k[:, :, t:t + n].copy(), stream_v[:, :, t:t + n].copy()
        st = cache.update(attn_state=(k, v), layer_idx=0, offset=n, cache_kwargs={"window_size": W})["attn_state"]
        out[f"hf_k_after_{i}"] = np.array(st[0], np.float32)
        out[f"hf_v_after_{i}"] = np.array(st[1], np.float32)
        t += n
    out["hf_steps"] = np.array(steps)
    out["hf_window"] = np.array(W)
    out["hf_stream_k"], out["hf_stream_v"] = stream_k, stream_v
    out["hf_seen_tokens"] = np.array(cache.get_seq_length(0))

    # 2. window block manager: prompts, decodes across block boundaries, a chunked prompt, a free
    bs, wl, nb = 16, 40, 24
    model = P.WindowCacheModel(nb, bs, wl)
    script = [("add", 0, 0, 0), ("prompt", 0, 70, 0), ("add", 1, 0, 0), ("prompt", 1, 5, 0)]
    script += [("decode", s, 1, 0) for _ in range(20) for s in (0, 1)]
    script += [("add", 2, 0, 0), ("prompt", 2, 33, 1), ("free", 0, 0, 0)]
    script += [("decode", s, 1, 0) for _ in range(18) for s in (1, 2)]
    slots = []
    for op, s, n, chunked in script:
        if op == "add":
            model.add_seq(s)
        elif op == "free":
            model.free_seq(s)
        else:
            slots += model.append_tokens(s, n, op == "prompt", store_all=bool(chunked))
    code = {"add": 0, "prompt": 1, "decode": 2, "free": 3}
    out["pg_script"] = np.array([[code[o], s, n, c] for o, s, n, c in script])
    out["pg_params"] = np.array([nb, bs, wl])
    out["pg_slots"] = np.array(slots, np.int64)
    out["pg_free"] = np.array(model.free)
    for s in (1, 2):
        table, n, first = model.view(s)
        out[f"pg_view_{s}"] = np.array(table + [n, first])

    # 3. paged decode attention, 7B head geometry in small: 2 sequences, GQA 4:2, window 32
    Hq, Hkv, D, bs = 4, 2, 128, 16
    lens = [37, 70]
    nblk = 8
    kc = bf16_bits(rng.standard_normal((nblk, bs, Hkv, D)).astype(np.float32))
    vc = bf16_bits(rng.standard_normal((nblk, bs, Hkv, D)).astype(np.float32))
    q = bf16_bits(rng.standard_normal((2, Hq, D)).astype(np.float32))
    tables = np.array([[5, 2, 7, 0, 0], [1, 6, 0, 3, 4]], np.int32)
    o, lse = A.paged_decode_attention(bf16_to_f32(q), bf16_to_f32(kc), bf16_to_f32(vc), tables, lens, D ** -0.5, 32,
                                      return_lse=True)
    out.update(dec_q=q, dec_k_cache=kc, dec_v_cache=vc, dec_tables=tables, dec_lens=np.array(lens, np.int32),
               dec_window_left=np.array(32), dec_out=o.astype(np.float32), dec_lse=lse.astype(np.float32))

    # 4. varlen prefill attention: two prompts (17 and 23 tokens), window 20
    qlens = [17, 23]
    T = sum(qlens)
    pq = bf16_bits(rng.standard_normal((T, Hq, D)).astype(np.float32))
    pk = bf16_bits(rng.standard_normal((T, Hkv, D)).astype(np.float32))
    pv = bf16_bits(rng.standard_normal((T, Hkv, D)).astype(np.float32))
    cu = np.concatenate([[0], np.cumsum(qlens)])
    po = A.varlen_window_attention(bf16_to_f32(pq), bf16_to_f32(pk), bf16_to_f32(pv), cu, cu, D ** -0.5, 20)
    out.update(pre_q=pq, pre_k=pk, pre_v=pv, pre_query_lens=np.array(qlens), pre_window_left=np.array(20),
               pre_out=po.astype(np.float32))

    # 5. GLA step: one (sequence, head); the whole updated state is summarised by row/column sums
    gq, gk, gv = (bf16_bits(rng.standard_normal((1, 1, D)).astype(np.float32)) for _ in range(3))
    gg = (-np.log1p(np.exp(-rng.standard_normal((1, 1, D)))) / 16).astype(np.float32)      # logsigmoid / 16
    state = (rng.standard_normal((1, 1, D, D)) * 0.02).astype(np.float32)
    st = state.astype(np.float64).copy()
    go = G.gla_step(bf16_to_f32(gq), bf16_to_f32(gk), bf16_to_f32(gv), gg, st)
    out.update(gla_q=gq, gla_k=gk, gla_v=gv, gla_g=gg, gla_state=state, gla_out=go.astype(np.float32),
               gla_state_rowsum=st[0, 0].sum(1).astype(np.float32), gla_state_colsum=st[0, 0].sum(0).astype(np.float32),
               gla_state_diag=np.diag(st[0, 0]).astype(np.float32))

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cache_path_v1.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes,", len(out), "arrays")
    write_extensions(np.random.default_rng(20240608))


def write_extensions(rng) -> None:
    """tests/golden/cache_path_v2_ext.npz: the paths added after v1 (its file stays byte-identical)."""
    from oracle import quant as Q

    out = {}
    D = 128
    # 6. per-row INT8: rows of different scales, an all-zero row, a tie row
    x = (rng.standard_normal((6, 2, D)) * rng.uniform(0.05, 8, (6, 2, 1))).astype(np.float32)
    x[1, 0] = 0
    x[2, 1, :4] = [127.0, 63.5, 62.5, -62.5]; x[2, 1, 4:] = 0
    xb = bf16_bits(x)
    codes, scale = Q.quantize_rows(bf16_to_f32(xb))
    out.update(i8_rows=xb, i8_codes=codes, i8_scales=scale, i8_dequant_bf16=Q.dequantize_rows(codes, scale, "bf16"))

    # 7. meta-token attention: 5 queries at the end of 9 keys, window 6, 8 meta tokens, their own 8 queries
    Hq, Hkv, M = 4, 2, 8
    q1 = bf16_bits(rng.standard_normal((5, Hq, D)).astype(np.float32))
    q2 = bf16_bits(rng.standard_normal((M, Hq, D)).astype(np.float32))
    k1, v1 = (bf16_bits(rng.standard_normal((9, Hkv, D)).astype(np.float32)) for _ in range(2))
    k2, v2 = (bf16_bits(rng.standard_normal((M, Hkv, D)).astype(np.float32)) for _ in range(2))
    mo = A.metatoken_attention(*(bf16_to_f32(t) for t in (q1, q2, k1, k2, v1, v2)), D ** -0.5, 6)
    out.update(mt_q1=q1, mt_q2=q2, mt_k1=k1, mt_v1=v1, mt_k2=k2, mt_v2=v2, mt_sliding_window=np.array(6),
               mt_out=mo.astype(np.float32))

    # 8. GLA over a 40-token prompt (one head): outputs and state summaries
    T = 40
    gq, gk, gv = (bf16_bits(np.maximum(rng.standard_normal((1, 1, T, D)), -0.5).astype(np.float32)) for _ in range(3))
    gg = (-np.log1p(np.exp(-rng.standard_normal((1, 1, T, D)))) / 16).astype(np.float32)
    s0 = (rng.standard_normal((1, 1, D, D)) * 0.02).astype(np.float32)
    go, gs = G.gla_recurrent(bf16_to_f32(gq), bf16_to_f32(gk), bf16_to_f32(gv), gg, s0.astype(np.float64))
    out.update(glp_q=gq, glp_k=gk, glp_v=gv, glp_g=gg, glp_state0=s0, glp_out=go.astype(np.float32),
               glp_state_rowsum=gs[0, 0].sum(1).astype(np.float32), glp_state_diag=np.diag(gs[0, 0]).astype(np.float32),
               glp_state_absmax=np.array(np.abs(gs).max(), np.float32))

    # 9. ragged paged decode (rows of 3, 150 and 40 keys, no window): the case the balanced split is for
    Hq, Hkv, bs = 4, 2, 16
    lens = [3, 150, 40]
    nblk = 16
    kc = bf16_bits(rng.standard_normal((nblk, bs, Hkv, D)).astype(np.float32))
    vc = bf16_bits(rng.standard_normal((nblk, bs, Hkv, D)).astype(np.float32))
    q = bf16_bits(rng.standard_normal((3, Hq, D)).astype(np.float32))
    tables = np.zeros((3, 10), np.int32)
    tables[0, :1] = [9]; tables[1, :10] = [4, 0, 11, 7, 2, 15, 6, 1, 13, 8]; tables[2, :3] = [3, 12, 5]
    o, lse = A.paged_decode_attention(bf16_to_f32(q), bf16_to_f32(kc), bf16_to_f32(vc), tables, lens, D ** -0.5, -1,
                                      return_lse=True)
    out.update(rag_q=q, rag_k_cache=kc, rag_v_cache=vc, rag_tables=tables, rag_lens=np.array(lens, np.int32),
               rag_out=o.astype(np.float32), rag_lse=lse.astype(np.float32))

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cache_path_v2_ext.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
