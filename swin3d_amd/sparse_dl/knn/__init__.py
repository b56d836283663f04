from .knn import KNN, knn_query

__all__ = ["KNN", "knn_query"]
