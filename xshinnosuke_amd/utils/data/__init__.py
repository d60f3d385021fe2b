"""DataSet / DataLoader (counterpart of xs/utils/data): seeded permutation, fixed batch tensors that are
re-sliced for a shorter last batch.  With ``device='cuda'`` the fixed tensors live on the device and every
batch is gathered into page-locked staging memory and uploaded with a copy that only enqueues on the stream."""
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
    def __init__(self, dataset, batch_size=None, shuffle=False, seed=None, device='cpu'):
        if device not in ('cpu', 'cuda'):
            raise ValueError("DataLoader: device must be 'cpu' or 'cuda'")
        self.device = device
        self.dataset = dataset
        n = len(dataset)
        self.batch_size = n if batch_size is None else min(int(batch_size), n)
        self.shuffle = shuffle
        self.seed = 0 if seed is None else seed
        self._order = None
        self._pos = 0
        if device == 'cuda':
            from ...backend import array as dev
            # device tensors hold float32 for floating data and the data's own type otherwise (labels)
            dts = [np.dtype(np.float32) if d.dtype.kind == 'f' else d.dtype for d in dataset.datas]
            self._pool = [Tensor(dev.empty((self.batch_size,) + d.shape[1:], dt)) for d, dt in zip(dataset.datas, dts)]
            # two sets of staging buffers: one is refilled while the upload from the other may still be in flight
            self._stage = [[dev.PinnedArray((self.batch_size,) + d.shape[1:], dt) for d, dt in zip(dataset.datas, dts)]
                           for _ in range(2)]
            self._uploaded = [None, None]
            self._flip = 0
        else:
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
        if self.device == 'cuda':
            from ...backend import array as dev
            k = self._flip
            self._flip ^= 1
            if self._uploaded[k] is not None:
                self._uploaded[k].synchronize()          # the upload that last read these staging buffers is done
            for t, d, pin in zip(self._pool, self.dataset.datas, self._stage[k]):
                t.slices(slice(None, len(sel), None) if len(sel) < self.batch_size else slice(None, None, None))
                pin.array[:len(sel)] = d[sel]
                t.eval.set_async(pin, len(sel))
                out.append(t)
            if self._uploaded[k] is None:
                self._uploaded[k] = dev.Event()
            self._uploaded[k].record()
            return out[0] if len(out) == 1 else out
        for t, d in zip(self._pool, self.dataset.datas):
            t.slices(slice(None, len(sel), None) if len(sel) < self.batch_size else slice(None, None, None))
            t.eval[...] = d[sel]
            out.append(t)
        return out[0] if len(out) == 1 else out
