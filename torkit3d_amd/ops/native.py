"""Pure-torch k nearest neighbours (API of torkit3d/ops/native.py): cdist + topk."""
import torch


def knn(query, key, k, sorted=False, transpose=False):
    """-> (knn_dist [B, N1, k] Euclidean distances, knn_ind [B, N1, k])."""
    if transpose:
        query, key = query.transpose(1, 2), key.transpose(1, 2)
    distance = torch.cdist(query, key)
    return torch.topk(distance, k, dim=2, largest=False, sorted=sorted)
