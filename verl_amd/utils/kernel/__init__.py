from .linear_cross_entropy import LinearCrossEntropy, linear_cross_entropy  # noqa: F401
