"""KV append kernel vs the oracle: bit-exact cache contents, sentinel bytes untouched."""
import numpy as np
import pytest
import torch

from oracle import paged as P

pytestmark = pytest.mark.gpu


def bits(t):
    return t.cpu().view(torch.int16 if t.element_size() == 2 else torch.int32).numpy()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("T,Hkv,D,bs,nb", [(64, 4, 128, 16, 40), (1, 4, 128, 16, 4), (333, 2, 64, 32, 30), (50, 8, 256, 16, 8)])
def test_append_bit_exact(sb, dev, dtype, T, Hkv, D, bs, nb):
    g = torch.Generator().manual_seed(T + D)
    key = torch.randn(T, Hkv, D, generator=g).to(dtype)
    val = torch.randn(T, Hkv, D, generator=g).to(dtype)
    slots = torch.randperm(nb * bs, generator=g)[:T].to(torch.int64)
    slots[torch.rand(T, generator=g) < 0.2] = -1
    kv = torch.full((2, nb, bs, Hkv, D), -3.0, dtype=dtype)
    exp_k, exp_v = kv[0].clone().numpy() if dtype == torch.float32 else kv[0].float().numpy(), None
    exp_k = kv[0].float().numpy().copy(); exp_v = kv[1].float().numpy().copy()
    P.kv_append(key.float().numpy(), val.float().numpy(), exp_k, exp_v, slots.tolist())
    kvd = kv.to(dev)
    sb.ops.kv_append(key.to(dev), val.to(dev), kvd[0], kvd[1], slots.to(dev))
    torch.cuda.synchronize()
    assert np.array_equal(kvd[0].float().cpu().numpy(), exp_k)
    assert np.array_equal(kvd[1].float().cpu().numpy(), exp_v)


def test_append_strided_views_of_a_fused_qkv(sb, dev):
    # key/value as the model hands them over: column slices of one [T, (Hq+2Hkv)*D] projection
    T, Hq, Hkv, D, bs, nb = 37, 28, 4, 128, 16, 8
    g = torch.Generator().manual_seed(1)
    qkv = torch.randn(T, (Hq + 2 * Hkv) * D, generator=g).bfloat16().to(dev)
    q, k, v = qkv.split([Hq * D, Hkv * D, Hkv * D], dim=-1)
    k, v = k.view(T, Hkv, D), v.view(T, Hkv, D)
    slots = torch.randperm(nb * bs, generator=g)[:T].to(torch.int64)
    kv = torch.zeros(2, nb, bs, Hkv, D, dtype=torch.bfloat16, device=dev)
    sb.ops.kv_append(k, v, kv[0], kv[1], slots.to(dev))
    exp_k = np.zeros((nb, bs, Hkv, D), np.float32); exp_v = exp_k.copy()
    P.kv_append(k.float().cpu().numpy(), v.float().cpu().numpy(), exp_k, exp_v, slots.tolist())
    assert np.array_equal(kv[0].float().cpu().numpy(), exp_k) and np.array_equal(kv[1].float().cpu().numpy(), exp_v)


def test_append_empty_and_all_padded(sb, dev):
    kv = torch.full((2, 4, 16, 4, 128), 5.0, dtype=torch.bfloat16, device=dev)
    e = torch.empty(0, 4, 128, dtype=torch.bfloat16, device=dev)
    sb.ops.kv_append(e, e, kv[0], kv[1], torch.empty(0, dtype=torch.int64, device=dev))
    k = torch.randn(3, 4, 128, device=dev).bfloat16()
    sb.ops.kv_append(k, k, kv[0], kv[1], torch.full((3,), -1, dtype=torch.int64, device=dev))
    torch.cuda.synchronize()
    assert (kv == 5.0).all()


def test_append_argument_errors(sb, dev):
    k = torch.zeros(2, 4, 128, dtype=torch.bfloat16, device=dev)
    cache = torch.zeros(4, 16, 4, 128, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError, match="int64"):
        sb.ops.kv_append(k, k, cache, cache, torch.zeros(2, dtype=torch.int32, device=dev))
    with pytest.raises(ValueError, match="share one dtype"):
        sb.ops.kv_append(k, k, cache.float(), cache.float(), torch.zeros(2, dtype=torch.int64, device=dev))
    with pytest.raises(ValueError):
        sb.ops.kv_append(k, k[:, :2], cache, cache, torch.zeros(2, dtype=torch.int64, device=dev))


def test_bulk_prefill_append_roundtrip_full_size(sb, dev):
    """BASELINE config 4's append: 16 x 8192 tokens, only the last 4096 of each sequence stored.
    Size-independent check: gathering the cache back through the slots returns the stored rows
    bit for bit, and unused blocks keep their sentinel."""
    n_seq, L, wl, Hkv, D, bs = 16, 8192, 4096, 4, 128, 16
    T = n_seq * L
    per_seq_blocks = wl // bs
    nb = n_seq * per_seq_blocks + 7
    g = torch.Generator().manual_seed(4)
    perm = torch.randperm(nb, generator=g)
    slots = torch.full((n_seq, L), -1, dtype=torch.int64)
    for s in range(n_seq):
        blocks = perm[s * per_seq_blocks:(s + 1) * per_seq_blocks]
        pos = torch.arange(L - wl, L)
        slots[s, L - wl:] = blocks[(pos - (L - wl)) // bs] * bs + pos % bs
    slots = slots.flatten().to(dev)
    key = torch.randn(T, Hkv, D, device=dev, dtype=torch.bfloat16)
    val = torch.randn(T, Hkv, D, device=dev, dtype=torch.bfloat16)
    kv = torch.full((2, nb, bs, Hkv, D), -1.0, dtype=torch.bfloat16, device=dev)
    sb.ops.kv_append(key, val, kv[0], kv[1], slots)
    stored = slots >= 0
    flat_k, flat_v = kv[0].view(nb * bs, Hkv, D), kv[1].view(nb * bs, Hkv, D)
    assert torch.equal(flat_k[slots[stored]], key[stored]) and torch.equal(flat_v[slots[stored]], val[stored])
    unused = perm[n_seq * per_seq_blocks:].to(dev)
    assert (kv[:, unused] == -1.0).all()
    assert int(stored.sum()) == n_seq * wl
