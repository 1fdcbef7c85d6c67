import torch


class SeedGenerator:
    """Mini-batch seed iterator over a node-id tensor (same contract as the
    reference's python/gs/utils/dataloader.py:4-44): optional reshuffle at the
    start of every pass, last partial batch kept unless drop_last."""

    def __init__(self, data: torch.Tensor, batch_size: int, shuffle: bool = False,
                 drop_last: bool = False):
        self.data = data
        self.batch_size = batch_size
        self.shuffle = shuffle
        self.drop_last = drop_last

    def __len__(self) -> int:
        n = self.data.shape[0]
        return n // self.batch_size if self.drop_last else -(-n // self.batch_size)

    def __iter__(self):
        if self.shuffle:
            perm = torch.randperm(self.data.shape[0], device=self.data.device)
            self.data = self.data[perm]
        self._step = 0
        self._last = len(self)
        return self

    def __next__(self) -> torch.Tensor:
        if self._step >= self._last:
            raise StopIteration
        lo = self._step * self.batch_size
        self._step += 1
        return self.data[lo:lo + self.batch_size].clone()
