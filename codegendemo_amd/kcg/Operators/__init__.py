"""Operator descriptions of the kcg mirror (matmul)."""
