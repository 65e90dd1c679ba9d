"""Weight layout for the bfloat16 MFMA kernels.

A matrix W [N, K] (out, in) is stored as tiles of 16 rows x 32 columns, each tile 1 KiB in the order in
which the 64 lanes of a wave hold the A/B operand of v_mfma_f32_16x16x32_bf16: lane = (k % 32) // 8 * 16 +
n % 16 holds the 8 elements k % 8.  Tiles of one 16-row band follow each other along K, bands follow each
other along N; N is padded to a multiple of 16 and K to a multiple of 32 with zeros.  A wave then reads its
operand with one fully contiguous 1 KiB load per tile and a whole band is one sequential stream, which is
what a decode step (bound by reading every weight once) wants."""
from __future__ import annotations

from dataclasses import dataclass

import torch

TILE_N, TILE_K = 16, 32


@dataclass
class PackedWeight:
    data: torch.Tensor      # bfloat16 [bands, chunks, 64, 8], contiguous
    N: int
    K: int

    @property
    def bands(self) -> int:
        return self.data.shape[0]

    @property
    def chunks(self) -> int:
        return self.data.shape[1]

    @property
    def shape(self):
        return (self.N, self.K)

    @property
    def dtype(self):
        return self.data.dtype

    @property
    def device(self):
        return self.data.device

    def nbytes(self) -> int:
        return self.data.numel() * self.data.element_size()


def pack_mfma(w: torch.Tensor) -> PackedWeight:
    """[N, K] bfloat16 -> the tiled layout (a new tensor)."""
    if w.dtype != torch.bfloat16 or w.dim() != 2:
        raise TypeError("pack_mfma takes a bfloat16 matrix")
    N, K = w.shape
    nb, kc = -(-N // TILE_N), -(-K // TILE_K)
    if nb * TILE_N != N or kc * TILE_K != K:
        padded = torch.zeros((nb * TILE_N, kc * TILE_K), dtype=w.dtype, device=w.device)
        padded[:N, :K] = w
        w = padded
    # [nb, 16, kc, 4, 8] -> [nb, kc, 4, 16, 8]: lane = c * 16 + i
    t = w.view(nb, TILE_N, kc, 4, 8).permute(0, 2, 3, 1, 4).contiguous()
    return PackedWeight(t.view(nb, kc, 64, 8), N, K)


def unpack_mfma(p: PackedWeight) -> torch.Tensor:
    nb, kc = p.bands, p.chunks
    t = p.data.view(nb, kc, 4, TILE_N, 8).permute(0, 3, 1, 2, 4).contiguous().view(nb * TILE_N, kc * TILE_K)
    return t[: p.N, : p.K].contiguous()


def can_pack(w: torch.Tensor) -> bool:
    return w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[1] % 8 == 0
