import torch


def recall(predict: torch.Tensor, target: torch.Tensor) -> float:
    """Mean per-row |predict ∩ target| / |target| over sets of ids
    (``pilot_ann/utils/recall.py:4-23``: rows are compared as sets, so a
    repeated id counts once)."""
    if not isinstance(predict, torch.Tensor):
        raise RuntimeError
    if not isinstance(target, torch.Tensor):
        raise RuntimeError
    if predict.size() != target.size():
        raise RuntimeError
    assert target.dim() == 2
    total = 0.0
    for y_hat, y in zip(predict.tolist(), target.tolist()):
        y = set(y)
        total += len(y.intersection(y_hat)) / len(y)
    return total / target.size(0)
