"""DataSet / DataLoader (counterpart of xs/utils/data): seeded permutation, fixed batch tensors that are
re-sliced for a shorter last batch."""
import numpy as np

from ...core.base import Tensor


class DataSet:
    def __init__(self, *datas):
        self.datas = [np.asarray(d) for d in datas]

    def __len__(self):
        return len(self.datas[0])

    def __getitem__(self, item):
        return [d[item] for d in self.datas]


class DataLoader:
    def __init__(self, dataset, batch_size=None, shuffle=False, seed=None):
        self.dataset = dataset
        n = len(dataset)
        self.batch_size = n if batch_size is None else min(int(batch_size), n)
        self.shuffle = shuffle
        self.seed = 0 if seed is None else seed
        self._order = None
        self._pos = 0
        self._pool = [Tensor(np.empty((self.batch_size,) + d.shape[1:], dtype=d.dtype)) for d in dataset.datas]
        self._reshuffle()

    def _reshuffle(self):
        n = len(self.dataset)
        if self.shuffle:
            self._order = np.random.RandomState(self.seed).permutation(n)
        else:
            self._order = np.arange(n)
        self._pos = 0

    def __len__(self):
        n = len(self.dataset)
        return (n + self.batch_size - 1) // self.batch_size

    def __iter__(self):
        return self

    def __next__(self):
        n = len(self.dataset)
        if self._pos >= n:
            self.seed += 1
            self._reshuffle()
            raise StopIteration
        sel = self._order[self._pos:self._pos + self.batch_size]
        self._pos += self.batch_size
        out = []
        for t, d in zip(self._pool, self.dataset.datas):
            t.slices(slice(None, len(sel), None) if len(sel) < self.batch_size else slice(None, None, None))
            t.eval[...] = d[sel]
            out.append(t)
        return out[0] if len(out) == 1 else out
