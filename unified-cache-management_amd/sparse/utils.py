"""Constants and the top-k length rule of the GSA path (ucm/sparse/utils.py:5-36)."""
from __future__ import annotations

DEFAULT_BLOCK_SIZE = 128
MIN_TOPK_LEN = 32
MAX_TOPK_LEN = 48
MAX_BS = 256
SEG_PREFILL_THRESHOLD = 8400
LOCAL_WINDOW_SZ = MIN_TOPK_LEN - 1
INIT_WINDOW_BLOCKS = 1   # ucm/sparse/gsa/offload_ops/include/select_topk_block.h:20
LOCAL_WINDOW_BLOCKS = 2


def round_up(x: int, y: int) -> int:
    return -(-x // y) * y


def compute_topk_len(raw_seq_len: int, min_len: int = MIN_TOPK_LEN, max_len: int = MAX_TOPK_LEN,
                     ratio: float = 0.3) -> int:
    """Blocks kept for a request of raw_seq_len blocks: 30 %, at least
    min(32, all of them), at most 48 - window blocks included."""
    k = int(raw_seq_len * ratio)
    if k < min_len:
        return min(min_len, raw_seq_len)
    return min(k, max_len)


class HeldBlocks:
    """The stored blocks one request's loads may read in place.  A store with a tier behind its pool moves blocks out
    of the pool when it runs short (``UcmHipBlockStore`` with ``host_spill_blocks``); the ones a kernel is going to
    read are held - brought back if they had left, and kept - from the first lookup until ``release``.  Any store
    with ``slot_of`` works; one without ``hold`` simply never moves its blocks."""

    def __init__(self, store):
        self.store = store
        self.held = set()

    def slots(self, hashes) -> list:
        """Pool block of every hash, -1 for one the store does not have."""
        hold = getattr(self.store, "hold", None)
        slot_of = self.store.slot_of
        if hold is None:
            return [slot_of.get(h, -1) for h in hashes]
        new = [h for h in dict.fromkeys(hashes) if h not in self.held]
        got = dict(zip(new, hold(new))) if new else {}
        self.held.update(h for h, s in got.items() if s >= 0)
        return [got[h] if h in got else slot_of.get(h, -1) for h in hashes]

    def release(self) -> None:
        release = getattr(self.store, "release", None)
        if release is not None and self.held:
            release(list(self.held))
        self.held.clear()
