"""Bit-packed HQMQ cache containers (device memory owned by torch).

PackedTensor holds one tensor (K or V) of one layer: the code planes, the
per-token scales, the Med3x flag plane and outlier sideband, and the joint
codebook the codes index.  PackedKV pairs a K and a V PackedTensor.
Plane layout: include/hqmq_amd.h.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from . import _lib as L

TILE = 16          # tokens per sideband tile
T_ALIGN = 64       # plane capacity is rounded up to whole attention super-tiles


def _round_up(x: int, m: int) -> int:
    return (x + m - 1) // m * m


class PackedTensor:
    """Packed codes of a (B, H, T, d_h) tensor; rows [0, length) are valid."""

    def __init__(self, B: int, H: int, t_cap: int, d_head: int, secondary_size: int, radius_bits: int,
                 dtype: torch.dtype, device, joint: Optional[torch.Tensor] = None, outliers: bool = False,
                 sideband_frac: float = 0.125, layout: Optional[tuple] = None):
        if d_head % 4:
            raise ValueError(f"d_head={d_head} not divisible by 4")
        self.B, self.H, self.d_head, self.n = B, H, d_head, d_head // 4
        self.d_head_orig = d_head            # smaller for zero-padded heads (PaddedHQMQ): what Q and O carry
        self.t_cap = _round_up(max(t_cap, 1), T_ALIGN)
        self.secondary_size, self.radius_bits = secondary_size, radius_bits
        self.qmax = (1 << radius_bits) - 1
        self.dtype, self.device = dtype, torch.device(device)
        # (idx_bits, main_bits, aux_bits); the default is the tight layout of include/hqmq_amd.h
        self.idx_bits, self.main_bits, self.aux_bits = layout or L.layout_bits(secondary_size, radius_bits)
        n = self.n
        z = dict(dtype=torch.uint8, device=self.device)
        self.main = torch.zeros(B, H, self.t_cap, (n * self.main_bits + 7) // 8, **z)
        self.aux = torch.zeros(B, H, self.t_cap, (n * self.aux_bits + 7) // 8, **z) if self.aux_bits else None
        self.scale = torch.zeros(B, H, self.t_cap, dtype=dtype, device=self.device)
        self.joint = joint
        # the largest finite scale written so far as fp32 bits (the quantize kernel keeps it up to date): the attention
        # kernels' range guard for bf16 / fp32 caches; fp16 scales cannot leave the range
        self.scale_max = None if dtype == torch.float16 else torch.zeros(1, dtype=torch.int32, device=self.device)
        # host-side copy of "scale_max lies outside [2^-8, 2^15)": such a cache takes the layout-generic attention kernel, which
        # guards the fp16 range (refresh_range reads the device value; the quantizer calls it after bulk appends and
        # every RANGE_CHECK_EVERY small ones)
        self.wide_range = False
        self._huge = False
        self._appends_since_range_check = 0
        self.length = 0                      # rows written when all sequences advance together
        self.lengths: Optional[torch.Tensor] = None  # per-sequence rows (int32, device) for ragged batches
        self.flags = self.sideband = self.sb_tile_off = self.sb_count = self.sb_overflow = self.sb_coord = None
        self.sb_cap = 0
        if outliers:
            self.flags = torch.zeros(B, H, self.t_cap, (n + 7) // 8, **z)
            self.sb_cap = max(64, int(self.t_cap * n * sideband_frac))
            self.sideband = torch.zeros(B, H, self.sb_cap, 4, dtype=dtype, device=self.device)
            # tiles not yet written read as "no entries"
            self.sb_tile_off = torch.full((B, H, self.t_cap // TILE), 0x7fffffff, dtype=torch.int32, device=self.device)
            self.sb_coord = torch.zeros(B, H, self.sb_cap, dtype=torch.int16, device=self.device)
            self.sb_count = torch.zeros(B, H, dtype=torch.int32, device=self.device)
            self.sb_overflow = torch.zeros(1, dtype=torch.int32, device=self.device)

    @property
    def has_outliers(self) -> bool:
        return self.flags is not None

    def row_bytes(self) -> float:
        """Stored bytes per (token, head), excluding sideband entries."""
        b = self.main.shape[-1] + self.scale.element_size()
        if self.aux is not None:
            b += self.aux.shape[-1]
        if self.flags is not None:
            b += self.flags.shape[-1]
        return b

    def nbytes(self, length: Optional[int] = None) -> int:
        """Algorithmic bytes of the first `length` rows of every (b, h) stream, sideband included."""
        t = self.length if length is None else length
        total = self.B * self.H * t * self.row_bytes()
        if self.sb_count is not None:
            total += int(self.sb_count.sum().item()) * 4 * self.scale.element_size()
        return int(total)

    def c_struct(self) -> L.Packed:
        s = L.Packed()
        s.main_plane, s.aux_plane, s.flag_plane = L.ptr(self.main), L.ptr(self.aux), L.ptr(self.flags)
        s.scale_plane = L.ptr(self.scale)
        s.scale_sb, s.scale_sh, s.scale_st = self.scale.stride(0), self.scale.stride(1), self.scale.stride(2)
        s.sideband, s.sb_tile_off, s.sb_cap = L.ptr(self.sideband), L.ptr(self.sb_tile_off), self.sb_cap
        s.sb_coord, s.sb_count = L.ptr(self.sb_coord), L.ptr(self.sb_count)
        s.joint, s.joint_sh, s.K = L.ptr(self.joint), self.joint.stride(0), self.joint.shape[1]
        s.scale_max_bits = L.ptr(self.scale_max)
        return s

    RANGE_CHECK_EVERY = 256     # small appends between two reads of the largest scale; set it to 1 (per cache or on the
                                # class) to read after every append: one device read each, and no window in which a bf16
                                # scale that left [2^-8, 2^15) still meets the unguarded kernels

    def refresh_range(self) -> bool:
        """Reads the largest scale written so far (one device read) and records whether it lies outside [2^-8, 2^15),
        the range inside which the specialised attention kernels keep P * (V scale) and the verbatim chunks in fp16's
        normal range.  The largest scale only grows: a cache of tiny values leaves the flag again when larger ones
        arrive; a cache beyond 2^15 keeps it."""
        if self.scale_max is not None and not self._huge:
            v = float(self.scale_max.view(torch.float32).item())
            self._huge = v >= 32768.0
            self.wide_range = self._huge or 0.0 < v < 2.0 ** -8
        self._appends_since_range_check = 0
        return self.wide_range

    def note_append(self, rows: int) -> None:
        """Called by the quantizer after an append of `rows` rows per sequence: bulk appends (a prefill) and every
        RANGE_CHECK_EVERY-th small one refresh the range flag; never while the stream is being captured."""
        if self.scale_max is None or self._huge:
            return
        self._appends_since_range_check += 1
        if (rows >= 64 or self._appends_since_range_check >= self.RANGE_CHECK_EVERY) and not torch.cuda.is_current_stream_capturing():
            self.refresh_range()

    def crop_(self, lengths) -> None:
        """Forgets the rows from `lengths` on (an int for all sequences or an int tensor [B]): the outlier list and
        its tile offsets go back to the state after the last kept row, so that the rows can be appended again.
        The planes themselves are left as they are (later appends overwrite them)."""
        B, H = self.B, self.H
        if isinstance(lengths, int):
            lens = torch.full((B,), lengths, dtype=torch.int64, device=self.device)
            self.length = min(self.length, lengths)
        else:
            lens = lengths.to(device=self.device, dtype=torch.int64).clamp(min=0)
            self.lengths = lens.to(torch.int32)
        if self.flags is None:
            return
        tiles = self.t_cap // TILE
        tile, r = lens // TILE, lens % TILE
        tc = tile.clamp(max=tiles - 1)
        off = self.sb_tile_off.gather(2, tc.view(B, 1, 1).expand(B, H, 1)).squeeze(2).to(torch.int64)
        # flagged chunks of the kept rows of the tile the cut falls into
        rows = tc.view(B, 1, 1) * TILE + torch.arange(TILE, device=self.device).view(1, 1, TILE)
        fl = self.flags.gather(2, rows.view(B, 1, TILE, 1).expand(B, H, TILE, self.flags.shape[-1]))
        bits = sum((fl >> i) & 1 for i in range(8)).to(torch.int64).sum(-1)                          # (B, H, TILE)
        kept = torch.arange(TILE, device=self.device).view(1, 1, TILE) < r.view(B, 1, 1)
        count = self.sb_count.to(torch.int64)
        new = torch.where((tile >= tiles).view(B, 1) | (off > count), count, off + (bits * kept).sum(-1))
        self.sb_count.copy_(torch.minimum(new, count).to(torch.int32))
        first_free = (lens + TILE - 1) // TILE             # tiles from here on hold no kept row: unwritten again
        gone = torch.arange(tiles, device=self.device).view(1, 1, tiles) >= first_free.view(B, 1, 1)
        self.sb_tile_off.masked_fill_(gone.expand(B, H, tiles), 0x7fffffff)
        dropped = torch.arange(self.t_cap, device=self.device).view(1, 1, self.t_cap, 1) >= lens.view(B, 1, 1, 1)
        self.flags.masked_fill_(dropped, 0)                # no flag without an entry behind it

    def with_fp8_table(self) -> "PackedTensor":
        """A view of the same planes whose joint table is rounded to float8_e4m3fn (kept in the table's dtype:
        every e4m3 number is exact there).  The rounded table is computed once per table."""
        import copy
        cached = getattr(self, "_fp8_view", None)
        if cached is None or cached[0] is not self.joint:
            view = copy.copy(self)
            view.joint = self.joint.to(torch.float8_e4m3fn).to(self.joint.dtype)
            cached = (self.joint, view)
            self._fp8_view = cached
        view = cached[1]
        view.length, view.lengths = self.length, self.lengths
        view.wide_range, view._huge = self.wide_range, self._huge
        return view

    def overflowed(self) -> bool:
        """True if an append found the sideband full (reads one int from the device).  The chunks that found no room
        were kept as plain HQMQ chunks (flag cleared, radius code written): nothing decodes to zero, the price is the
        accuracy of those chunks."""
        return self.sb_overflow is not None and bool(int(self.sb_overflow.item()))

    def check_overflow(self) -> None:
        """Raises if an append ran out of sideband room (see overflowed)."""
        if self.overflowed():
            raise L.HqmqError(f"outlier sideband overflow: more than {self.sb_cap} flagged chunks in one (b, h) stream "
                              "(the chunks beyond it were stored as plain HQMQ chunks); allocate the cache with a larger "
                              "sideband_frac")


@dataclass
class PackedKV:
    """The compressed K and V of one layer."""
    K: PackedTensor
    V: PackedTensor

    @property
    def length(self) -> int:
        return self.K.length

    def nbytes(self, length: Optional[int] = None) -> int:
        return self.K.nbytes(length) + self.V.nbytes(length)

    def crop_(self, lengths) -> None:
        """Forgets the rows from `lengths` on in K and V (see PackedTensor.crop_)."""
        self.K.crop_(lengths)
        self.V.crop_(lengths)
