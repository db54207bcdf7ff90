"""flash_trittention for MI355X (gfx950): 3-way attention on hand-written HIP kernels.

Same public names as the reference package (src/flash_trittention/__init__.py:11-14):
``flash_trittention`` (triple-dot-product) and ``TrittentionTriton``
(dot-product-sum; the name is kept so imports drop in — there is no Triton
inside), plus ``FlashTrittentionModule``, an ``nn.Module`` front of the former.  Imports are lazy so ``import flash_trittention`` works without a GPU.
"""

__version__ = "0.1.0"

__all__ = ["flash_trittention", "TrittentionTriton", "FlashTrittentionModule"]

_LAZY = {
    "flash_trittention": (".triple_dot_product.flash_trittention", "flash_trittention"),
    "TrittentionTriton": (".dot_product_sum.trittention_triton", "TrittentionTriton"),
    "FlashTrittentionModule": (".triple_dot_product.flash_trittention", "FlashTrittentionModule"),
}


def __getattr__(name):
    if name not in _LAZY:
        raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
    from importlib import import_module

    mod, attr = _LAZY[name]
    value = getattr(import_module(mod, __name__), attr)
    globals()[name] = value
    return value


def __dir__():
    return sorted(list(globals()) + list(_LAZY))
