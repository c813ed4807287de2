"""Caller-side memory in named HBM regions (`nbo_alloc_placed`, a measurement entry point): two
or three flat device buffers, each wholly inside one of the regions the placement search tells
apart -- or, with -1 for every buffer, rotating over the regions as the optimizer's state does --
to measure what such placement of a framework's parameter and gradient storage would buy
(`python -m nabla_amd.kernel_bench --placed`: nothing, -3 to +0 %).  `regions` gives a region number per
buffer: equal numbers share a region, different numbers lie in different regions."""
from __future__ import annotations

import ctypes as C
from typing import List, Sequence, Tuple

from . import _lib
from .optim import _call


class _Span:
    """A device address range as an object torch can wrap (the CUDA array interface)."""

    def __init__(self, ptr: int, nbytes: int, owner):
        self.__cuda_array_interface__ = {"shape": (nbytes,), "typestr": "|u1", "data": (ptr, False), "version": 2}
        self._owner = owner  # keeps the allocation alive as long as a tensor made from this lives


class PlacedBuffers:
    def __init__(self, nbytes: int, regions: Sequence[int]):
        n = len(regions)
        self._h = C.c_void_p()
        ptrs = (C.c_void_p * 3)()
        _call(_lib.load().nbo_alloc_placed(n, int(nbytes), (C.c_int * n)(*regions), ptrs, C.byref(self._h)))
        self.nbytes = int(nbytes)
        self.ptrs = [int(ptrs[k]) for k in range(n)]

    def note(self) -> str:
        buf = C.create_string_buffer(512)
        _call(_lib.load().nbo_placed_note(self._h, buf, 512))
        return buf.value.decode()

    def bytes_tensor(self, k: int):
        """Buffer k as a flat uint8 tensor on cuda:0 (aliases the buffer; keep this object alive)."""
        import torch

        return torch.as_tensor(_Span(self.ptrs[k], self.nbytes, self), device="cuda:0")

    def carve(self, k: int, shapes: Sequence[Tuple[int, int]], dtype) -> List:
        """Tensors of the given shapes laid out one after the other in buffer k, each starting
        at a multiple of 256 bytes."""
        import torch

        flat = self.bytes_tensor(k)
        item = torch.empty((), dtype=dtype).element_size()
        out, off = [], 0
        for r, c in shapes:
            nb = r * c * item
            if off + nb > self.nbytes:
                raise ValueError("the shapes do not fit the buffer")
            out.append(flat[off:off + nb].view(dtype).view(r, c))
            off = (off + nb + 255) // 256 * 256
        return out

    def close(self) -> None:
        if self._h:
            _call(_lib.load().nbo_free_placed(self._h))
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def carved_bytes(shapes: Sequence[Tuple[int, int]], item_bytes: int) -> int:
    """Bytes `PlacedBuffers.carve` needs for these shapes."""
    off = 0
    for r, c in shapes:
        off = (off + r * c * item_bytes + 255) // 256 * 256
    return max(off, 256)
