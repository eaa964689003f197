"""Arrays between sentinel-filled guard regions, and packed offsets that are inconsistent in every way a device-side
``cu_seqlens`` can be: what the bounds tests hand to the kernels."""

import torch

GUARD = 4096  # bytes on either side of every array
SENTINEL = 0xA5


class Arena:
    """Arrays carved out of one device buffer, each surrounded by sentinel bytes."""

    def __init__(self, dev):
        self.dev = dev
        self.items = []

    def make(self, n, dtype, fill=None):
        esize = torch.empty((), dtype=dtype).element_size()
        raw = torch.full((GUARD + n * esize + GUARD,), SENTINEL, dtype=torch.uint8, device=self.dev)
        view = raw[GUARD:GUARD + n * esize].view(dtype)
        if fill is not None:
            view.copy_(fill.to(self.dev))
        self.items.append((raw, n * esize))
        return view

    def guards_intact(self):
        for raw, nbytes in self.items:
            head, tail = raw[:GUARD], raw[GUARD + nbytes:]
            if not (bool((head == SENTINEL).all()) and bool((tail == SENTINEL).all())):
                return False
        return True


BAD_OFFSETS = {
    # N = 100 tokens, B = 3 sequences
    "last_beyond_the_arrays": [0, 30, 60, 5000],
    "last_short_of_the_arrays": [0, 30, 60, 90],
    "first_not_zero": [5, 30, 60, 100],
    "negative": [-50, 30, 60, 100],
    "decreasing": [0, 70, 40, 100],
    "huge": [0, 30, 2**40, 100],
    "all_beyond": [1000, 2000, 3000, 4000],
}
