"""Constants of the INT8-X codec and of the deploy helpers.

The numeric tables restate the reference's ``ixrun/config.py:21-51`` (level
scheme, code offsets, skip list, minimum layer size, decode block size); the
Windows paths of that file are not part of the hot path and are left out.
"""
from __future__ import annotations

import torch

# (3,5,8): |v|<=3 in 3 bits, 3<|v|<=15 in 5 bits, the rest in 8 bits
# (reference ixrun/config.py:21).
DEFAULT_LEVELS = (3, 5, 8)

# A b-bit level stores the signed values [-T_b, T_b] as the unsigned code
# v + T_b with T_b = 2**(b-1) - 1 (reference ixrun/config.py:27-36).
BIT_TO_THRESHOLD = {b: (1 << (b - 1)) - 1 for b in range(1, 9)}

# Linear layers whose dotted name contains one of these stay unquantized
# (reference ixrun/config.py:39), as do layers under MIN_LINEAR_ELEMS weights
# (reference ixrun/config.py:42).
SKIP_PATTERNS = ("lm_head", "embed", "shared", "wte", "wte_emb")
MIN_LINEAR_ELEMS = 1000

CUDA = torch.device("cuda:0") if torch.cuda.is_available() else torch.device("cpu")
CPU = torch.device("cpu")

# Flat elements per entry of the block-offset tables returned by
# precompute_block_offsets (reference ixrun/config.py:51).
TRITON_BLOCK = 1024
