from .knn import KNN, KNNInterpolate, knn_interpolate, knn_max_pool, knn_query

__all__ = ["KNN", "KNNInterpolate", "knn_interpolate", "knn_max_pool", "knn_query"]
