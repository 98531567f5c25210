"""Pins oracle.attention against a library routine (torch SDPA) and against special cases the
mathematics fixes."""
import numpy as np
import torch
import torch.nn.functional as F

from oracle import attention as A


def rng(seed):
    return np.random.default_rng(seed)


def test_mask_is_W_keys_including_self_bottom_right_aligned():
    m = ~A.sliding_causal_mask(3, 7, 3)  # allowed
    # queries sit at absolute positions 4, 5, 6; each sees itself and the two keys before it
    assert [np.nonzero(r)[0].tolist() for r in m] == [[2, 3, 4], [3, 4, 5], [4, 5, 6]]
    assert (~A.sliding_causal_mask(1, 5, 100))[0].all()          # window wider than the cache: all keys
    assert (~A.sliding_causal_mask(4, 4, 1)).sum() == 4           # W=1: only self


def test_repeat_kv_matches_repeat_interleave():
    x = rng(0).standard_normal((2, 4, 5, 3))
    np.testing.assert_array_equal(A.repeat_kv(x, 7), np.repeat(x, 7, axis=1))


def test_sdpa_window_attention_vs_torch_sdpa_with_left_padding():
    B, Hq, Hkv, Q, K, D, W = 3, 8, 2, 5, 11, 16, 4
    r = rng(1)
    q = r.standard_normal((B, Hq, Q, D)); k = r.standard_normal((B, Hkv, K, D)); v = r.standard_normal((B, Hkv, K, D))
    am = np.ones((B, K + 2), np.int64); am[1, :5] = 0; am[2, :9] = 0      # left padding, row 2 pads into the queries
    got = A.sdpa_window_attention(q, k, v, W, am)
    kp = np.arange(K); qa = (K - Q) + np.arange(Q)
    allowed = (kp[None] <= qa[:, None]) & (kp[None] > qa[:, None] - W)
    mask = (~allowed)[None, None] | (am[:, -K:] == 0)[:, None, None, :]
    add = torch.where(torch.from_numpy(mask), -torch.inf, 0.0).double()
    ref = F.scaled_dot_product_attention(torch.from_numpy(q), torch.from_numpy(np.repeat(k, Hq // Hkv, 1)),
                                         torch.from_numpy(np.repeat(v, Hq // Hkv, 1)), attn_mask=add)
    ref = torch.nan_to_num(ref, nan=0.0).numpy()
    np.testing.assert_allclose(got, ref, rtol=1e-10, atol=1e-12)
    assert (got[2, :, :1] == 0).all() and (got[2, :, 1:] != 0).any()   # the pad query of row 2 is fully masked -> zeros


def dense_reference(q, kk, vv, scale, window_left):
    """torch SDPA on one sequence's gathered keys; q [Hq, D], kk/vv [n, Hkv, D]."""
    n, Hkv, D = kk.shape
    Hq = q.shape[0]
    i = np.arange(n)
    masked = i < (n - 1 - window_left) if window_left >= 0 else np.zeros(n, bool)
    add = torch.where(torch.from_numpy(masked), -torch.inf, 0.0).double()[None, None, None, :]
    kr = torch.from_numpy(np.repeat(kk.transpose(1, 0, 2), Hq // Hkv, 0))[None]
    vr = torch.from_numpy(np.repeat(vv.transpose(1, 0, 2), Hq // Hkv, 0))[None]
    return F.scaled_dot_product_attention(torch.from_numpy(q)[None, :, None, :], kr, vr, attn_mask=add,
                                          scale=scale)[0, :, 0].numpy()


def make_paged(B, lens, bs, Hkv, D, seed, nb_extra=5):
    r = rng(seed)
    need = [(n + bs - 1) // bs for n in lens]
    nb = sum(need) + nb_extra
    perm = r.permutation(nb)
    kc = r.standard_normal((nb, bs, Hkv, D)); vc = r.standard_normal((nb, bs, Hkv, D))
    tables = np.zeros((B, max(need)), np.int32)
    p = 0
    for b in range(B):
        tables[b, :need[b]] = perm[p:p + need[b]]; p += need[b]
    return kc, vc, tables


def test_paged_decode_vs_torch_sdpa_on_gathered_keys():
    B, Hq, Hkv, D, bs, wl = 4, 14, 2, 16, 16, 20
    lens = [1, 17, 48, 50]
    kc, vc, tables = make_paged(B, lens, bs, Hkv, D, 2)
    q = rng(3).standard_normal((B, Hq, D))
    out, lse = A.paged_decode_attention(q, kc, vc, tables, lens, 0.3, wl, return_lse=True)
    for b, n in enumerate(lens):
        kk = np.concatenate([kc[t] for t in tables[b]])[:n]   # independent gather: concatenate blocks in order
        vv = np.concatenate([vc[t] for t in tables[b]])[:n]
        np.testing.assert_allclose(out[b], dense_reference(q[b], kk, vv, 0.3, wl), rtol=1e-10, atol=1e-12)
        lo = max(0, n - 1 - wl)
        s = np.einsum("hd,nhd->hn", q[b].reshape(Hkv, -1, D).reshape(Hq, D), np.repeat(kk, Hq // Hkv, 1))[:, lo:] * 0.3
        np.testing.assert_allclose(lse[b], np.log(np.exp(s).sum(1)), rtol=1e-10)


def test_paged_decode_special_cases_and_invariants():
    B, Hq, Hkv, D, bs = 2, 4, 2, 8, 16
    lens = [40, 33]
    kc, vc, tables = make_paged(B, lens, bs, Hkv, D, 4)
    q = rng(5).standard_normal((B, Hq, D))
    # window_left = 0: only the newest key is visible -> output is exactly that V row
    out = A.paged_decode_attention(q, kc, vc, tables, lens, 1.0, 0)
    for b, n in enumerate(lens):
        vrow = vc[tables[b, (n - 1) // bs], (n - 1) % bs]
        np.testing.assert_allclose(out[b], np.repeat(vrow, Hq // Hkv, 0), rtol=1e-12)
    # constant V -> constant output whatever the scores
    vconst = np.full_like(vc, 2.5)
    np.testing.assert_allclose(A.paged_decode_attention(q, kc, vconst, tables, lens, 1.0, 12), 2.5, rtol=1e-12)
    # relabelling physical blocks (permute cache rows, rewrite the table) changes nothing
    nb = kc.shape[0]
    perm = rng(6).permutation(nb)
    inv = np.argsort(perm)
    base = A.paged_decode_attention(q, kc, vc, tables, lens, 0.5, 12)
    moved = A.paged_decode_attention(q, kc[perm], vc[perm], inv[tables].astype(np.int32), lens, 0.5, 12)
    np.testing.assert_allclose(moved, base, rtol=1e-12)
    # a wider window never loses keys: window >= n equals unbounded
    np.testing.assert_allclose(A.paged_decode_attention(q, kc, vc, tables, lens, 0.5, 1000),
                               A.paged_decode_attention(q, kc, vc, tables, lens, 0.5, -1), rtol=1e-12)


def test_varlen_vs_torch_sdpa_and_decode_consistency():
    Hq, Hkv, D, wl = 4, 2, 8, 5
    cu_q = [0, 6, 6, 9]; cu_k = [0, 6, 10, 21]          # seq0: plain prompt; seq1: no queries; seq2: 3 new of 11
    r = rng(7)
    q = r.standard_normal((9, Hq, D)); k = r.standard_normal((21, Hkv, D)); v = r.standard_normal((21, Hkv, D))
    out = A.varlen_window_attention(q, k, v, cu_q, cu_k, 0.4, wl)
    for s in range(3):
        Lq, Lk = cu_q[s + 1] - cu_q[s], cu_k[s + 1] - cu_k[s]
        for j in range(Lq):
            n = Lk - Lq + j + 1                            # this query as a decode over the first n keys
            ref = dense_reference(q[cu_q[s] + j], k[cu_k[s]:cu_k[s] + n], v[cu_k[s]:cu_k[s] + n], 0.4, wl)
            np.testing.assert_allclose(out[cu_q[s] + j], ref, rtol=1e-10, atol=1e-12)


def test_soft_cap_and_alibi_vs_torch_and_limits():
    """The two flash-attn options of the backend (meta_attention.py:665-690). ALiBi against torch SDPA with
    the bias written out as an additive mask; the soft cap against its limits (a huge cap changes nothing,
    a vanishing cap flattens the scores: the output is the mean of the visible V rows) and against the
    formula evaluated by torch on explicit scores."""
    B, Hq, Hkv, D, bs, wl = 3, 6, 2, 16, 16, 20
    lens = [1, 30, 50]
    kc, vc, tables = make_paged(B, lens, bs, Hkv, D, 12)
    q = rng(13).standard_normal((B, Hq, D))
    slopes = [2.0 ** -(i + 1) for i in range(Hq)]
    G = Hq // Hkv
    out = A.paged_decode_attention(q, kc, vc, tables, lens, 0.3, wl, alibi_slopes=slopes)
    capped = A.paged_decode_attention(q, kc, vc, tables, lens, 0.3, wl, softcap=1.5)
    both = A.paged_decode_attention(q, kc, vc, tables, lens, 0.3, wl, softcap=1.5, alibi_slopes=slopes)
    for b, n in enumerate(lens):
        kk = np.concatenate([kc[t] for t in tables[b]])[:n]
        vv = np.concatenate([vc[t] for t in tables[b]])[:n]
        i = np.arange(n)
        vis = i >= n - 1 - wl
        kr = torch.from_numpy(np.repeat(kk.transpose(1, 0, 2), G, 0))      # [Hq, n, D]
        vr = torch.from_numpy(np.repeat(vv.transpose(1, 0, 2), G, 0))
        dist = torch.from_numpy((n - 1 - i).astype(np.float64))
        add = torch.where(torch.from_numpy(vis), 0.0, -torch.inf).double()[None, :] - torch.tensor(slopes).double()[:, None] * dist[None, :]
        ref = F.scaled_dot_product_attention(torch.from_numpy(q[b])[None, :, None, :], kr[None], vr[None],
                                             attn_mask=add[None, :, None, :], scale=0.3)[0, :, 0].numpy()
        np.testing.assert_allclose(out[b], ref, rtol=1e-10, atol=1e-12)
        sc = torch.einsum("hd,hnd->hn", torch.from_numpy(q[b]), kr) * 0.3
        for cap, bias, got in ((1.5, 0.0, capped[b]), (1.5, 1.0, both[b])):
            logits = cap * torch.tanh(sc / cap) - bias * torch.tensor(slopes).double()[:, None] * dist[None, :]
            logits = torch.where(torch.from_numpy(vis)[None, :], logits, -torch.inf)
            ref2 = torch.einsum("hn,hnd->hd", torch.softmax(logits, -1), vr).numpy()
            np.testing.assert_allclose(got, ref2, rtol=1e-10, atol=1e-12)
        flat = A.paged_decode_attention(q, kc, vc, tables, lens, 0.3, wl, softcap=1e-9)[b]
        np.testing.assert_allclose(flat, np.repeat(vv[vis].mean(0), G, 0), rtol=1e-6)
    np.testing.assert_allclose(A.paged_decode_attention(q, kc, vc, tables, lens, 0.3, wl, softcap=1e9),
                               A.paged_decode_attention(q, kc, vc, tables, lens, 0.3, wl), rtol=1e-9)
    # the varlen form: every query is a decode over the keys up to its own position, options included
    cu_q = [0, 5, 9]; cu_k = [0, 5, 17]
    r = rng(14)
    qv = r.standard_normal((9, Hq, D)); kv = r.standard_normal((17, Hkv, D)); vv_ = r.standard_normal((17, Hkv, D))
    got = A.varlen_window_attention(qv, kv, vv_, cu_q, cu_k, 0.4, 6, softcap=2.0, alibi_slopes=slopes)
    for s_ in range(2):
        Lq, Lk = cu_q[s_ + 1] - cu_q[s_], cu_k[s_ + 1] - cu_k[s_]
        for j in range(Lq):
            n = Lk - Lq + j + 1
            kc1 = kv[cu_k[s_]:cu_k[s_] + n][None]; vc1 = vv_[cu_k[s_]:cu_k[s_] + n][None]   # one block of n rows
            one = A.paged_decode_attention(qv[cu_q[s_] + j][None], kc1, vc1, np.zeros((1, 1), np.int32), [n], 0.4, 6,
                                           softcap=2.0, alibi_slopes=slopes)
            np.testing.assert_allclose(got[cu_q[s_] + j], one[0], rtol=1e-10, atol=1e-12)


def test_lse_merge_equals_attention_over_union():
    D, nA, nB = 8, 5, 7
    r = rng(8)
    q = r.standard_normal((3, D)); kA = r.standard_normal((nA, D)); vA = r.standard_normal((nA, D))
    kB = r.standard_normal((nB, D)); vB = r.standard_normal((nB, D))
    none = np.zeros((1, 1), bool)
    oA, lA = A.masked_softmax_attention(q, kA, vA, none, 0.5, return_lse=True)
    oB, lB = A.masked_softmax_attention(q, kB, vB, none, 0.5, return_lse=True)
    oU, lU = A.masked_softmax_attention(q, np.concatenate([kA, kB]), np.concatenate([vA, vB]), none, 0.5, return_lse=True)
    o, l = A.lse_merge(oA, lA, oB, lB)
    np.testing.assert_allclose(o, oU, rtol=1e-10)
    np.testing.assert_allclose(l, lU, rtol=1e-10)


def test_metatoken_attention_is_window_attention_merged_with_meta_attention():
    """The one-softmax statement (fa_kernel_metatoken.py:372-405) against the two-attention +
    log-sum-exp merge the flash path runs (:124-194): pins both to the same mathematics; also the
    closed case of no cached keys visible beyond the meta tokens."""
    r = rng(21)
    Hq, Hkv, D, M, Lk, Lq, W = 4, 2, 8, 6, 11, 3, 5
    q1 = r.standard_normal((Lq, Hq, D)); q2 = r.standard_normal((M, Hq, D))
    k1 = r.standard_normal((Lk, Hkv, D)); v1 = r.standard_normal((Lk, Hkv, D))
    k2 = r.standard_normal((M, Hkv, D)); v2 = r.standard_normal((M, Hkv, D))
    out = A.metatoken_attention(q1, q2, k1, k2, v1, v2, 0.3, W)
    assert out.shape == (Lq + M, Hq, D)
    G = Hq // Hkv
    none = np.zeros((1, 1), bool)
    for h in range(Hq):
        for i in range(Lq):
            pos = Lk - Lq + i
            ks = slice(max(0, pos - W + 1), pos + 1)
            oa, la = A.masked_softmax_attention(q1[i:i + 1, h], k1[ks, h // G], v1[ks, h // G], none, 0.3, return_lse=True)
            ob, lb = A.masked_softmax_attention(q1[i:i + 1, h], k2[:, h // G], v2[:, h // G], none, 0.3, return_lse=True)
            o, _ = A.lse_merge(oa, la, ob, lb)
            np.testing.assert_allclose(out[i, h], o[0], rtol=1e-10)
        om = A.masked_softmax_attention(q2[:, h], k2[:, h // G], v2[:, h // G], none, 0.3)
        np.testing.assert_allclose(out[Lq:, h], om, rtol=1e-10)
    # meta values all equal to c and a query orthogonal to every window key: result between c and the window average
    v2c = np.full_like(v2, 2.0)
    k1z = np.zeros_like(k1)
    k2z = np.zeros_like(k2)
    o = A.metatoken_attention(q1, None, k1z, k2z, np.full_like(v1, 5.0), v2c, 0.3, W)
    # equal scores everywhere: M meta tokens (value 2) and min(W, pos+1) window keys (value 5)
    for i in range(Lq):
        n = min(W, Lk - Lq + i + 1)
        np.testing.assert_allclose(o[i], (2.0 * M + 5.0 * n) / (M + n), rtol=1e-12)


def test_flash_window_attention_is_W_plus_one_keys_and_unpads():
    """flash window_size=(W, 0) = the query and W keys to its left. Constant scores make the output the
    mean of the visible V rows, which names them; pads (a prefix) are invisible and pad queries give 0.
    Against the SDPA-flavour oracle it is the same mask one key wider."""
    B, H, K, D, W = 2, 1, 8, 4, 2
    q = np.zeros((B, H, K, D)); k = np.zeros((B, H, K, D))
    v = np.broadcast_to(np.arange(K, dtype=np.float64)[None, None, :, None], (B, H, K, D)).copy()
    am = np.ones((B, K + 1), np.int64); am[1, :4] = 0          # row 1: positions 0..2 of the keys are pads
    out = A.flash_window_attention(q, k, v, W, am)
    # row 0, query i sees keys max(0, i-2)..i
    np.testing.assert_allclose(out[0, 0, :, 0], [0, 0.5, 1, 2, 3, 4, 5, 6])
    # row 1: keys 3..7 are real; queries 0..2 are pads -> zeros; query 3 sees {3}, 4 {3,4}, 5 {3,4,5}, 6 {4,5,6}
    np.testing.assert_allclose(out[1, 0, :, 0], [0, 0, 0, 3, 3.5, 4, 5, 6])
    # decode shape: one query at the end of K keys sees the last W+1 real keys
    np.testing.assert_allclose(A.flash_window_attention(q[:, :, -1:], k, v, W, am)[:, 0, 0, 0], [6, 6])
    r = rng(5)
    q = r.standard_normal((B, 4, K, D)); k = r.standard_normal((B, 2, K, D)); v = r.standard_normal((B, 2, K, D))
    np.testing.assert_allclose(A.flash_window_attention(q, k, v, W, am), A.sdpa_window_attention(q, k, v, W + 1, am),
                               rtol=1e-12, atol=1e-12)


def test_metatoken_attention_with_soft_cap_and_alibi_vs_torch_two_attention_form():
    """Score options together with meta tokens, against torch running the flash path's own form
    (fa_kernel_metatoken.py:235-279): a causal sliding-window attention per sequence with the ALiBi term
    -slope * (pos_q - key) written out as an additive mask, a second NON-causal attention of all stacked query
    rows (every sequence's tokens, then the meta tokens' own queries) over the meta keys whose ALiBi term is
    flash-attn's -slope * |i + M - N - j| for stacked row i of N, both with the cap softcap * tanh(x / softcap)
    on the scaled scores first, merged by log-sum-exp. Two sequences, so that the stacked index differs from
    the index inside a sequence."""
    import torch
    r = rng(33)
    Hq, Hkv, D, M, W, cap = 4, 2, 8, 5, 4, 1.7
    G = Hq // Hkv
    scale = 0.35
    slopes = [0.5, 0.25, 0.125, 0.0625]
    lens = [(3, 9), (4, 4)]                      # (new tokens, keys) of the two sequences
    N = sum(lq for lq, _ in lens) + M            # rows of the stacked second attention
    k2 = r.standard_normal((M, Hkv, D)); v2 = r.standard_normal((M, Hkv, D))
    q2 = r.standard_normal((M, Hq, D))
    seqs = [(r.standard_normal((lq, Hq, D)), r.standard_normal((lk, Hkv, D)), r.standard_normal((lk, Hkv, D))) for lq, lk in lens]

    def attend(q, k, v, bias, masked):           # torch: capped, biased, masked scores -> (out, lse)
        s = torch.tensor(q) @ torch.tensor(k).T * scale
        s = cap * torch.tanh(s / cap) + torch.tensor(bias)
        s = s.masked_fill(torch.tensor(masked), float("-inf"))
        return (torch.softmax(s, -1) @ torch.tensor(v)).numpy(), torch.logsumexp(s, -1).numpy()

    row0 = 0
    for si, (q1, k1, v1) in enumerate(seqs):
        lq, lk = lens[si]
        got = A.metatoken_attention(q1, q2 if si == 0 else None, k1, k2, v1, v2, scale, W, softcap=cap, alibi_slopes=slopes,
                                    stack_row0=row0, stack_rows=N)
        pos = lk - lq + np.arange(lq)
        keys = np.arange(lk)
        dist = pos[:, None] - keys[None, :]
        masked = (dist < 0) | (dist >= W)
        stacked = row0 + np.arange(lq)
        for h in range(Hq):
            oa, la = attend(q1[:, h], k1[:, h // G], v1[:, h // G], -slopes[h] * dist, masked)
            mb = -slopes[h] * np.abs(stacked[:, None] + M - N - np.arange(M)[None, :])
            ob, lb = attend(q1[:, h], k2[:, h // G], v2[:, h // G], mb, np.zeros((lq, M), bool))
            o, _ = A.lse_merge(oa, la, ob, lb)
            np.testing.assert_allclose(got[:lq, h], o, rtol=1e-9, atol=1e-12)
            if si == 0:                          # the meta tokens' own queries: the last M stacked rows, meta keys only
                st2 = N - M + np.arange(M)
                mb2 = -slopes[h] * np.abs(st2[:, None] + M - N - np.arange(M)[None, :])
                o2, _ = attend(q2[:, h], k2[:, h // G], v2[:, h // G], mb2, np.zeros((M, M), bool))
                np.testing.assert_allclose(got[lq:, h], o2, rtol=1e-9, atol=1e-12)
        row0 += lq
    # a slope of zero and a huge cap change nothing
    q1, k1, v1 = seqs[0]
    plain = A.metatoken_attention(q1, None, k1, k2, v1, v2, scale, W)
    same = A.metatoken_attention(q1, None, k1, k2, v1, v2, scale, W, softcap=1e9, alibi_slopes=[0.0] * Hq, stack_rows=N)
    np.testing.assert_allclose(same, plain, rtol=1e-9)
