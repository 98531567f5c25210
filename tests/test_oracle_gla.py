"""Pins oracle.gla against what the mathematics fixes: the unrolled closed form of the
recurrence, special cases, in-place slot semantics."""
import numpy as np

from oracle import gla


def rand(shape, seed):
    return np.random.default_rng(seed).standard_normal(shape)


def test_unrolled_closed_form():
    # S_T = diag(exp(sum_u g_u)) S_0 + sum_t diag(exp(sum_{u>t} g_u)) k_t^T v_t ; o_T = scale * q_T S_T
    B, H, T, D = 2, 3, 7, 8
    q, k, v = rand((B, H, T, D), 0), rand((B, H, T, D), 1), rand((B, H, T, D), 2)
    g = -np.abs(rand((B, H, T, D), 3)) * 0.3
    S0 = rand((B, H, D, D), 4) * 0.1
    o, ST = gla.gla_recurrent(q, k, v, g, initial_state=S0, scale=0.37)
    for b in range(B):
        for h in range(H):
            for T_ in (1, 4, T):
                S = np.exp(g[b, h, :T_].sum(0))[:, None] * S0[b, h]
                for t in range(T_):
                    decay = np.exp(g[b, h, t + 1:T_].sum(0))
                    S = S + decay[:, None] * np.outer(k[b, h, t], v[b, h, t])
                np.testing.assert_allclose(o[b, h, T_ - 1], 0.37 * q[b, h, T_ - 1] @ S, rtol=1e-12, atol=1e-12)
                if T_ == T:
                    np.testing.assert_allclose(ST[b, h], S, rtol=1e-12, atol=1e-12)


def test_special_cases():
    B, H, D = 2, 2, 8
    q, k, v = rand((B, H, D), 0), rand((B, H, D), 1), rand((B, H, D), 2)
    S0 = rand((B, H, D, D), 3)
    # g = 0: pure accumulation
    S = S0.copy()
    gla.gla_step(q, k, v, np.zeros((B, H, D)), S, scale=1.0)
    np.testing.assert_allclose(S, S0 + k[..., :, None] * v[..., None, :])
    # k = 0: pure decay of rows by exp(g) (per KEY dim = per row of S)
    g = -np.abs(rand((B, H, D), 4))
    S = S0.copy()
    gla.gla_step(q, np.zeros_like(k), v, g, S, scale=1.0)
    np.testing.assert_allclose(S, np.exp(g)[..., :, None] * S0)
    # q = e_i / scale reads row i of the UPDATED state
    S = S0.copy()
    e = np.zeros((B, H, D)); e[..., 3] = 1 / 0.25
    o = gla.gla_step(e, k, v, g, S, scale=0.25)
    np.testing.assert_allclose(o, S[..., 3, :])
    # default scale is D^-0.5
    S1, S2 = S0.copy(), S0.copy()
    np.testing.assert_allclose(gla.gla_step(q, k, v, g, S1), gla.gla_step(q, k, v, g, S2, scale=D ** -0.5))


def test_slots_in_place_and_skip():
    B, H, D, slots = 3, 2, 4, 5
    q, k, v = rand((B, H, D), 0), rand((B, H, D), 1), rand((B, H, D), 2)
    g = -np.abs(rand((B, H, D), 3))
    state = rand((slots, H, D, D), 4)
    before = state.copy()
    o = gla.gla_step(q, k, v, g, state, slot_idx=[4, -1, 0])
    assert np.isnan(o[1]).all() and not np.isnan(o[[0, 2]]).any()      # skipped row is never written
    np.testing.assert_array_equal(state[[1, 2, 3]], before[[1, 2, 3]])  # untouched slots
    exp4 = np.exp(g[0])[..., :, None] * before[4] + k[0][..., :, None] * v[0][..., None, :]
    np.testing.assert_allclose(state[4], exp4)
    # same rows through identity slots on a copy give the same numbers (in place == out of place)
    s2 = before[[4, 0]].copy()
    o2 = gla.gla_step(q[[0, 2]], k[[0, 2]], v[[0, 2]], g[[0, 2]], s2)
    np.testing.assert_allclose(o2, o[[0, 2]])
    np.testing.assert_allclose(s2, state[[4, 0]])
