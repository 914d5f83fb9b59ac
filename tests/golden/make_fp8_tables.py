"""Writes the exhaustive bf16 -> fp8 code tables used as golden fixtures.

For every one of the 65536 bf16 bit patterns b, table[b] is the byte PyTorch's
CPU cast produces for `bf16_value.to(torch.float8_e4m3fn)` / `.to(torch.float8_e5m2)`.
These are the casts the reference applies in `x.div(s).to(fp8)`; the tables pin
the quantisers of the oracle, of oracle/fp8_codec.c and of the HIP kernels.

Run from the repository root:  python tests/golden/make_fp8_tables.py
"""
import pathlib

import numpy as np
import torch

here = pathlib.Path(__file__).parent
bits = torch.arange(65536, dtype=torch.int32).to(torch.uint16)
vals = bits.view(torch.bfloat16)
for name, dt in (("bf16_to_e4m3fn", torch.float8_e4m3fn), ("bf16_to_e5m2", torch.float8_e5m2)):
    codes = vals.to(dt).view(torch.uint8).numpy()
    assert codes.shape == (65536,)
    (here / f"{name}.bin").write_bytes(codes.tobytes())
    print(name, "sha1-ish sum", int(codes.astype(np.uint64).sum()))
