from typing import Optional


def process_masking_variables(seq_len: int, k1_window: Optional[int] = None, k2_window: Optional[int] = None,
                              kk_left: Optional[int] = None, kk_right: Optional[int] = None):
    """``None`` means "no window" = seq_len (reference triple_dot_product/kernels/utils.py:6-17)."""
    f = lambda w: seq_len if w is None else int(w)
    return f(k1_window), f(k2_window), f(kk_left), f(kk_right)
