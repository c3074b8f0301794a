"""Sign-random-projection hash codes on the GPU kernels.

Same surface as the reference's ``HashEncoder``
(ucm/sparse/kvcomp/hash_encoder.py:35-219): weights drawn N(0, std 2) of shape
``[input_dim, hash_bits]`` (:65-71), ``set_hash_weight`` (:76-90),
``compute_hash(x) -> uint8 [..., hash_bits // 8]`` with bit j of byte b = column
8b+j, LSB first, strict ``> 0`` (:92-97, :139-149), ``_unpack_hash`` to +-1 fp16
(:159-219).

The reference multiplies with ``torch.matmul`` and keeps the sign of whatever
that library's accumulation order gives; here the projection runs on the matrix
cores and every sign is that of the exactly accumulated product (results within
rounding of zero are redone in fp64), so codes do not depend on a GEMM's
summation order.  The kernels are built for ``input_dim == hash_bits == 128`` in
bfloat16 or float16 (the model's type: keys, queries and weights alike); anything
else is refused, there is no other path.
"""
from __future__ import annotations

from typing import Optional

import torch

from ... import ops


class HashEncoder:
    def __init__(self, input_dim: int, hash_bits: int, dtype: torch.dtype, device: torch.device) -> None:
        if hash_bits % 8 != 0:
            raise ValueError("hash_bits must be a multiple of 8")
        if input_dim != 128 or hash_bits != 128:
            raise ValueError(f"the hash kernels are built for input_dim = hash_bits = 128, got {input_dim} / {hash_bits}")
        if dtype not in (torch.bfloat16, torch.float16):
            raise ValueError(f"the hash kernels take bfloat16 or float16 keys, queries and weights, got {dtype}")
        self.input_dim, self.hash_bits = input_dim, hash_bits
        self.hash_numbers = hash_bits // 8
        self.dtype, self.device = dtype, torch.device(device)
        if self.device.type != "cuda":
            raise ValueError("HashEncoder needs a GPU device")
        self.hash_weights = torch.normal(mean=0, std=2, size=(input_dim, hash_bits), dtype=dtype, device=self.device)
        self.bit_masks = torch.pow(2, torch.arange(8, dtype=torch.uint8, device=self.device)).view(1, 1, 8)

    def set_hash_weight(self, hash_weights: torch.Tensor) -> None:
        if hash_weights.shape != (self.input_dim, self.hash_bits):
            raise ValueError(f"hash_weights shape {hash_weights.shape} does not match required shape "
                             f"{(self.input_dim, self.hash_bits)}")
        if hash_weights.dtype != self.dtype:
            raise ValueError(f"hash_weights dtype {hash_weights.dtype} does not match required dtype {self.dtype}")
        if hash_weights.device != self.device:
            raise ValueError(f"hash_weights device {hash_weights.device} does not match required device {self.device}")
        self.hash_weights.copy_(hash_weights)

    def compute_hash(self, x: torch.Tensor) -> torch.Tensor:
        """x [..., input_dim] -> uint8 [..., hash_numbers].  Any leading shape: the vectors are
        handed to the block kernel as blocks of 32 one-head tokens (the tail is zero-padded)."""
        if x.shape[-1] != self.input_dim:
            raise ValueError(f"x must be of shape (..., {self.input_dim}), but got {x.shape}")
        if x.device != self.device:
            raise ValueError(f"x device {x.device} does not match required device {self.device}")
        lead = x.shape[:-1]
        flat = x.reshape(-1, self.input_dim)
        if flat.dtype != self.dtype:
            flat = flat.to(self.dtype)
        n = flat.shape[0]
        if n == 0:
            return torch.empty(lead + (self.hash_numbers,), dtype=torch.uint8, device=self.device)
        n_blocks = (n + 31) // 32
        if n_blocks * 32 != n or not flat.is_contiguous():
            padded = torch.zeros((n_blocks * 32, self.input_dim), dtype=self.dtype, device=self.device)
            padded[:n] = flat
            flat = padded
        pool = flat.view(n_blocks, 32, 1, self.input_dim)
        codes = torch.empty((1, n_blocks, 32, 1, self.hash_numbers), dtype=torch.uint8, device=self.device)
        colsum = torch.empty((1, n_blocks, 1, self.hash_bits), dtype=torch.int16, device=self.device)
        bcodes = torch.empty((1, n_blocks, 1, self.hash_numbers), dtype=torch.uint8, device=self.device)
        ops.hash_encode_blocks(ops.LayerPointers([pool]), None, None, n_blocks, self.hash_weights, 32, 1, n_blocks,
                               colsum, bcodes, token_codes=codes)
        return codes.view(-1, self.hash_numbers)[:n].reshape(lead + (self.hash_numbers,))

    def encode_cache_blocks(self, k_layers: "ops.LayerPointers", block_ids: torch.Tensor, slots: torch.Tensor,
                            block_size: int, kv_heads: int, num_blocks: int, colsum: torch.Tensor,
                            block_codes: torch.Tensor, token_codes: Optional[torch.Tensor] = None) -> None:
        """What ``compute_hash(k_cache[ids])`` feeds (kvcomp.py:320-323), read straight from the paged
        cache: token codes (optional), per-(head, bit) column sums and majority codes of each block."""
        ops.hash_encode_blocks(k_layers, block_ids, slots, block_ids.numel(), self.hash_weights, block_size, kv_heads,
                               num_blocks, colsum, block_codes, token_codes=token_codes)

    def _unpack_hash(self, packed_codes: torch.Tensor) -> torch.Tensor:
        if packed_codes.shape[-1] != self.hash_numbers:
            raise ValueError(f"packed_codes must be of shape (..., {self.hash_numbers}), but got {packed_codes.shape}")
        if packed_codes.device != self.device:
            raise ValueError(f"packed_codes device {packed_codes.device} does not match required device {self.device}")
        if packed_codes.dtype != torch.uint8:
            raise ValueError(f"packed_codes dtype {packed_codes.dtype} is not torch.uint8")
        lead = packed_codes.shape[:-1]
        bits = (packed_codes.reshape(-1, self.hash_numbers, 1) & self.bit_masks) > 0
        return (bits.to(torch.float16) * 2 - 1).view(lead + (self.hash_bits,))
