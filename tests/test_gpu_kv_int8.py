"""Per-row INT8 K/V: codes and scales bit-exact against the oracle (integer/byte work), decode
attention over the INT8 cache within 2e-2 of the oracle's attention over the dequantised rows."""
import numpy as np
import pytest
import torch

from oracle import attention as A
from oracle import quant as Q

pytestmark = pytest.mark.gpu

D = 128


def rows(T, H, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, D, generator=g) * (10 ** torch.empty(T, H, 1).uniform_(-3, 2, generator=g))
    x[0, 0] = 0                                  # scale clamps to 1e-5
    if T > 2:
        x[1, 0, :3] = torch.tensor([3e6, -3e6, 1.5e4])   # scale clamps to 1e4, codes saturate
        x[2, 0, :4] = torch.tensor([127.0, 63.5, 62.5, -62.5]); x[2, 0, 4:] = 0   # ties
    return x.to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("H", [4, 2, 7])
def test_append_int8_bit_exact(sb, dev, dtype, H):
    nb, bs, T = 9, 16, 40
    k, v = rows(T, H, 1, dtype), rows(T, H, 2, dtype)
    g = torch.Generator().manual_seed(3)
    slots = torch.randperm(nb * bs, generator=g)[:T]
    slots[5] = -1
    kv, sc = sb.ops.alloc_int8_kv_cache(nb, bs, H, D, dev)
    kv.fill_(3); sc.fill_(-1.0)
    ref_kv = kv.cpu().numpy().copy(); ref_sc = sc.cpu().numpy().copy()
    Q.kv_append_int8(k.float().numpy(), v.float().numpy(), ref_kv[0], ref_kv[1], ref_sc[0], ref_sc[1], slots.tolist())
    # token-major views of a fused projection, as the layers produce them
    fused = torch.cat([k, v], 1).to(dev)
    sb.ops.kv_append_int8(fused[:, :H], fused[:, H:], kv[0], kv[1], sc[0], sc[1], slots.to(dev))
    assert np.array_equal(kv.cpu().numpy(), ref_kv)
    assert np.array_equal(sc.cpu().numpy(), ref_sc)


@pytest.mark.parametrize("dtype,name", [(torch.bfloat16, "bf16"), (torch.float16, "f16"), (torch.float32, "f32")])
def test_quantize_sym_bit_exact(sb, dev, dtype, name):
    x = rows(33, 4, 7, dtype)
    ref = Q.quantize_sym(x.float().numpy(), name)
    xd = x.to(dev)
    y = sb.ops.quantize_sym(xd)
    assert np.array_equal(y.float().cpu().numpy(), ref)
    sb.ops.quantize_sym(xd, out=xd)              # in place
    assert torch.equal(xd, y)
