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
