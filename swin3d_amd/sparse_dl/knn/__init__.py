from .knn import KNN, KNNInterpolate, knn_interpolate, knn_query

__all__ = ["KNN", "KNNInterpolate", "knn_interpolate", "knn_query"]
