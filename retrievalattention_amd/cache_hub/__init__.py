from .kmeans import segment_k_means
from .retroinfer_cache import retroinfer_cache
