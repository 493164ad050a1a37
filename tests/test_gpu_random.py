"""Seeded random shapes of the attention operators against the CPU oracle: sequence lengths around the
tile sizes (1, 63..65, 127..129, 255..257, ...), different query and key lengths, both dtypes and head
dims, index widths, explicit sample lists, smooth blocks longer than the sequence."""
import math
import random

import pytest
import torch

from oracle import hyper_oracle as O
from _util import _gen, _randn, assert_close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ha():
    import hyperattention_amd
    return hyperattention_amd


def _causal_reference(q, k, v):
    """Exact attention with the kernel's (and src/flash_attn_triton.py:147-149's) top-left aligned
    causal mask for different query and key lengths: query i sees keys 0..i."""
    d = q.shape[-1]
    s = (q.double() @ k.double().transpose(-1, -2)) / math.sqrt(d)
    mask = torch.arange(k.shape[2])[None, :] > torch.arange(q.shape[2])[:, None]
    s = s.masked_fill(mask, float("-inf"))
    return torch.softmax(s, -1) @ v.double(), torch.logsumexp(s, -1)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_flash_random_shapes(ha, seed):
    rnd = random.Random(seed)
    for it in range(25):
        dtype = rnd.choice([torch.float16, torch.bfloat16])
        d, b, h = rnd.choice([64, 128]), rnd.choice([1, 2]), rnd.choice([1, 2, 3])
        nq = rnd.choice([1, 7, 63, 64, 65, 127, 200, 255, 256, 257, 300, 511, 513, 777, 1025])
        nk = nq if rnd.random() < 0.5 else rnd.choice([1, 5, 64, 100, 129, 256, 300, 640, 1000])
        causal = rnd.random() < 0.5
        print(f"flash seed={seed} case={it} {dtype} d={d} b={b} h={h} nq={nq} nk={nk} causal={causal}", flush=True)
        q = _randn((b, h, nq, d), 1000 * seed + it, dtype)
        k, v = (_randn((b, h, nk, d), 1000 * seed + s + it, dtype) for s in (100, 200))
        o, lse = ha.flash_attn_func(q.cuda().transpose(1, 2), k.cuda().transpose(1, 2), v.cuda().transpose(1, 2),
                                    None, causal, None)
        ro, rl = _causal_reference(q, k, v) if causal else O.exact_attention(q, k, v)
        assert_close(o.transpose(1, 2), ro, "flash out", dtype)
        assert_close(lse[:, :, :nq], rl, "flash lse")


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_block_attention_random_shapes(ha, seed):
    rnd = random.Random(100 + seed)
    for it in range(20):
        dtype = rnd.choice([torch.float16, torch.bfloat16])
        d, b, h = rnd.choice([64, 128]), rnd.choice([1, 2]), rnd.choice([1, 2, 3])
        n = 128 * rnd.choice([1, 2, 3, 5, 8, 9, 16])
        block = rnd.choice([128, 256, 384, 512])
        sample = min(rnd.choice([0, 128, 256]), n)
        smooth = rnd.random() < 0.5
        idt = rnd.choice([torch.int32, torch.int64])
        g = _gen(5000 * seed + it)
        q, k, v = (_randn((b, h, n, d), 5000 * seed + s + it, dtype) for s in (100, 200, 300))
        qi = torch.sort(torch.randint(0, 16, (b, h, n), generator=g), dim=2, stable=True)[1]
        ki = torch.sort(torch.randint(0, 16, (b, h, n), generator=g), dim=2, stable=True)[1]
        sidx = torch.randint(0, n, (sample,), generator=g) if (sample and rnd.random() < 0.5) else None
        print(f"block seed={seed} case={it} {dtype} d={d} b={b} h={h} n={n} block={block} sample={sample} "
              f"smooth={smooth} idx={idt} explicit_samples={sidx is not None}", flush=True)
        c = lambda t: t.cuda()
        o, lse = ha.hyper_attn_func(c(q).transpose(1, 2), c(k).transpose(1, 2), c(v).transpose(1, 2),
                                    c(qi).to(idt).transpose(1, 2), c(ki).to(idt).transpose(1, 2), block, sample,
                                    None, smooth, sampled_idx=None if sidx is None else c(sidx))
        ro, rl = O.block_sampled_attention(q, k, v, qi, ki, block, sample, None, smooth, sidx)
        assert_close(o.transpose(1, 2), ro, "block out", dtype)
        assert_close(lse, rl, "block lse")
