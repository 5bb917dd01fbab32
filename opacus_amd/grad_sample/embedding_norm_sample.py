"""Import location kept from the reference (opacus/grad_sample/embedding_norm_sample.py)."""

from .embedding import compute_embedding_norm_sample  # noqa: F401
