from .pi3_sparse_like import Pi3SparseLike  # noqa: F401
