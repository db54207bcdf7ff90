from typing import Optional


def process_masking_variables(seq_len: int, k1_window: Optional[int] = None, k2_window: Optional[int] = None,
                              kk_left: Optional[int] = None, kk_right: Optional[int] = None):
    """``None`` means "no window" = seq_len (reference triple_dot_product/kernels/utils.py:6-17).

    Values are clamped to seq_len (a window that wide excludes nothing, and the C ABI takes 32-bit ints:
    an unclamped 2**32 would wrap to 0); a negative window raises ValueError."""
    return tuple(clamp_window(w, seq_len, n) for w, n in
                 ((k1_window, "k1_window"), (k2_window, "k2_window"), (kk_left, "kk_left"), (kk_right, "kk_right")))


def clamp_window(w: Optional[int], seq_len: int, name: str = "window") -> int:
    if w is None:
        return seq_len
    w = int(w)
    if w < 0:
        raise ValueError(f"{name} must be non-negative or None, got {w}")
    return min(w, seq_len)
