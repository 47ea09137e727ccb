"""Cache and state manager of the ragged-step engine.

Two kinds of per-sequence memory, both owned here and handed to the layers as plain device tensors:
  * PAGED planes: something a layer keeps for EVERY token of a sequence (an attention layer's cached rows).  One pool of page ids is
    shared by all planes, so a sequence has one page table; a plane is a tensor (pages, page_size, *row_shape).
  * SLOT states: something of fixed size per sequence (a recurrent layer's state, a convolution's last inputs, a token-shift row).
    A state is a tensor (slots, *shape); a slot is cleared when a sequence takes it, so a new sequence starts from zeros.
Pages and slots go back to the free lists when a sequence is released and are handed out again, lowest id first.
"""
import torch

from ._lib import ZLError


class CacheManager:
    def __init__(self, max_tokens, max_seqs, device, page_size=64):
        if max_tokens <= 0 or max_seqs <= 0 or page_size <= 0:
            raise ZLError("the cache needs max_tokens, max_seqs and page_size > 0")
        self.page_size, self.device = page_size, torch.device(device)
        self.n_pages = (max_tokens + page_size - 1) // page_size
        self.n_slots = max_seqs
        self.free_pages = list(range(self.n_pages))
        self.free_slots = list(range(self.n_slots))
        self.planes, self.states = {}, {}
        self.seqs = {}                      # id -> {"slot", "pages", "len"}

    # ---- what layers register ------------------------------------------------------------------
    def add_plane(self, name, row_shape, dtype):
        if name in self.planes:
            raise ZLError(f"cache plane {name} exists")
        t = torch.zeros((self.n_pages, self.page_size) + tuple(row_shape), dtype=dtype, device=self.device)
        self.planes[name] = t
        return t

    def add_state(self, name, shape, dtype=torch.float32):
        if name in self.states:
            raise ZLError(f"state {name} exists")
        t = torch.zeros((self.n_slots,) + tuple(shape), dtype=dtype, device=self.device)
        self.states[name] = t
        return t

    # ---- sequences -----------------------------------------------------------------------------
    def admit(self, sid):
        if sid in self.seqs:
            raise ZLError(f"sequence {sid} is live already")
        if not self.free_slots:
            raise ZLError("no free state slot")
        slot = self.free_slots.pop(0)
        for t in self.states.values():      # a fill kernel per state (no memset node: a caller may capture the step)
            t[slot].zero_()
        self.seqs[sid] = {"slot": slot, "pages": [], "len": 0}
        return slot

    def can_extend(self, sid, count):
        s = self.seqs.get(sid)
        have = len(s["pages"]) if s else 0
        length = s["len"] if s else 0
        return (length + count + self.page_size - 1) // self.page_size - have <= len(self.free_pages)

    def extend(self, sid, count):
        """room for `count` more tokens; returns (pos0, slot, pages) of the portion and advances the sequence's length"""
        s = self.seqs[sid]
        need = (s["len"] + count + self.page_size - 1) // self.page_size - len(s["pages"])
        if need > len(self.free_pages):
            raise ZLError("the page pool is exhausted")
        for _ in range(need):
            s["pages"].append(self.free_pages.pop(0))
        pos0 = s["len"]
        s["len"] += count
        return pos0, s["slot"], s["pages"]

    def length(self, sid):
        return self.seqs[sid]["len"]

    def release(self, sid):
        s = self.seqs.pop(sid)
        self.free_pages = sorted(self.free_pages + s["pages"])
        self.free_slots = sorted(self.free_slots + [s["slot"]])

    def live(self):
        return list(self.seqs)
