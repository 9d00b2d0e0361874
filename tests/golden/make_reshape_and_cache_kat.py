"""Writes tests/golden/reshape_and_cache_kat.npz: the one CPU-reproducible known-answer case the
reference holds (benchmark/test_reshape_and_cache.py:29-42 of the reference: torch.manual_seed(42)
on the CPU, 4 tokens of 8 heads x 128, slots [6, 134, 212, 290], caches [583, 64, 128, 16]).

The inputs are the reference's (same seed, same draw order: key, value, then the key of the
key-only case).  The expected placement is written out as explicit (block, offset) pairs and flat
element positions computed here with integer arithmetic only -- block = slot // 128,
offset = slot % 128, element f of a token's row at [block, f // 16, offset, f % 16] -- so the
fixture does not depend on any function it is later used to check.

Run from the repository root:  python tests/golden/make_reshape_and_cache_kat.py
"""
import os

import numpy as np
import torch

torch.manual_seed(42)
slots = np.array([6, 134, 212, 290], dtype=np.int32)
key = torch.randn(4, 8, 128, dtype=torch.float16)
value = torch.randn(4, 8, 128, dtype=torch.float16)
key2 = torch.randn(4, 8, 128, dtype=torch.float16)
P, C = 128, 64
blocks = slots // P
offsets = slots % P
f = np.arange(8 * 128)
# flat index into a [583, 64, 128, 16] cache of element f of token t
flat = (blocks[:, None].astype(np.int64) * C + f[None, :] // 16) * P * 16 + offsets[:, None] * 16 + f[None, :] % 16
out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reshape_and_cache_kat.npz")
np.savez_compressed(
    out,
    slots=slots,
    key_bits=key.view(torch.int16).numpy(),
    value_bits=value.view(torch.int16).numpy(),
    key2_bits=key2.view(torch.int16).numpy(),
    blocks=blocks.astype(np.int32),
    offsets=offsets.astype(np.int32),
    flat_index=flat,
    cache_shape=np.array([583, 64, 128, 16], dtype=np.int32),
)
print(out, blocks.tolist(), offsets.tolist())
