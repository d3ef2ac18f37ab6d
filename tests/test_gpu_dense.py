"""The dense fp16 baseline kernels against the oracle's dense attention (model/Llama_AlignedKV.py:130-139)."""
import numpy as np
import pytest
import torch

from oracle import akv_oracle as O
from tests.common import make_qkv

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("B,H,L,steps", [(2, 4, 300, 3), (1, 8, 1, 40), (2, 2, 1023, 2)])
def test_dense_step_matches_oracle(B, H, L, steps):
    from alignedkv_amd.dense_baseline import DenseKVCache
    D = 128
    q, k, v = make_qkv(B, L + steps, H, D, seed=L, n_outliers=0)
    rng = np.random.default_rng(L)
    c = DenseKVCache(B, L + steps + 5, H, D)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    c.prefill(dev(k[:, :L]), dev(v[:, :L]))
    for t in range(L, L + steps):
        qt = rng.standard_normal((B, 1, H, D)).astype(np.float16)
        out = c.decode(dev(qt), dev(k[:, t:t + 1]), dev(v[:, t:t + 1]))
        want = O.dense_attention(qt, k[:, :t + 1], v[:, :t + 1])
        assert np.max(np.abs(out.cpu().numpy().astype(np.float32) - want.astype(np.float32))) <= 2e-3
    assert torch.equal(c.k[:, :, :L + steps].transpose(1, 2).cpu(), torch.from_numpy(k))
