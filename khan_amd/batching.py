"""Host batch assembly and device feeding for the featurizer.

`RawDataset` mirrors khan/data/dataset.py:7-183: molecules are ragged arrays of rows (type, x, y, z), a
batch is their concatenation plus, per atom, the index of its molecule inside the batch; the last
batch is not padded (dataset.py:118-183).

`DeviceFeeder` is what the reference does with a feed dict and a staging queue
(khan/training/trainer_multi_tower.py:767-792, 291-303), done for one GPU with PyTorch as the memory
and stream plumbing: it splits a batch into the flat arrays the ops take (xs, ys, zs, atom types,
molecule indices), copies them through pinned host buffers with asynchronous host-to-device copies on a
side stream, runs `mol_offsets` and `ani_sort` on the device, and keeps one batch in flight while the
caller works on the previous one.
"""
import math

import numpy as np


class RawDataset:
    """Ragged molecules [(n_i, 4) arrays of (type, x, y, z)], optional labels and per-atom gradients."""

    def __init__(self, all_Xs, all_ys=None, all_grads=None):
        self.all_Xs = list(all_Xs)
        self.all_ys = None if all_ys is None else list(all_ys)
        self.all_grads = None if all_grads is None else list(all_grads)
        if self.all_ys is not None and len(self.all_ys) != len(self.all_Xs):
            raise ValueError("all_ys must have one entry per molecule")
        if self.all_grads is not None and len(self.all_grads) != len(self.all_Xs):
            raise ValueError("all_grads must have one entry per molecule")

    def num_mols(self):
        return len(self.all_Xs)

    def num_batches(self, batch_size):
        return math.ceil(self.num_mols() / batch_size)

    def iterate(self, batch_size, shuffle, fuzz=None, rng=None):
        """Yields (mol_Xs [N,4], mol_ids [N], mol_yts or None, mol_grads [N,3] or None) per batch.

        mol_ids[a] is the position of atom a's molecule inside the batch.  `fuzz` adds uniform noise in
        [-fuzz, fuzz] to the coordinates (dataset.py:166-169).  `rng` is a numpy Generator (the reference
        draws from numpy's global state)."""
        rng = np.random.default_rng() if rng is None else rng
        perm = np.arange(self.num_mols())
        if shuffle:
            rng.shuffle(perm)
        for batch_idx in range(self.num_batches(batch_size)):
            sel = perm[batch_idx * batch_size:min((batch_idx + 1) * batch_size, self.num_mols())]
            mols = [np.asarray(self.all_Xs[p]) for p in sel]
            mol_ids = np.repeat(np.arange(len(sel), dtype=np.int32), [len(m) for m in mols])
            mol_Xs = np.concatenate(mols, axis=0) if mols else np.zeros((0, 4))
            if fuzz is not None:
                mol_Xs = mol_Xs.copy()
                mol_Xs[:, 1:4] += rng.uniform(-fuzz, fuzz, (mol_Xs.shape[0], 3))
            mol_yts = None if self.all_ys is None else [self.all_ys[p] for p in sel]
            mol_grads = None
            if self.all_grads is not None:
                mol_grads = np.concatenate([np.asarray(self.all_grads[p]) for p in sel], axis=0)
            yield mol_Xs, mol_ids, mol_yts, mol_grads


def split_columns(mol_Xs, mol_ids, dtype=np.float32):
    """(type, x, y, z) rows -> the flat arrays the ops take: xs, ys, zs [N] dtype; atom types, mol ids int32
    (trainer_multi_tower.py:769-779)."""
    mol_Xs = np.asarray(mol_Xs)
    return (np.ascontiguousarray(mol_Xs[:, 1], dtype=dtype), np.ascontiguousarray(mol_Xs[:, 2], dtype=dtype),
            np.ascontiguousarray(mol_Xs[:, 3], dtype=dtype), np.ascontiguousarray(mol_Xs[:, 0]).astype(np.int32),
            np.ascontiguousarray(mol_ids, dtype=np.int32))


class DeviceBatch:
    """One batch resident on the GPU, with everything `featurize` needs."""

    __slots__ = ("xs", "ys", "zs", "atom_types", "mol_idxs", "n_mols", "mol_atom_counts", "mol_offsets",
                 "scatter_idxs", "gather_idxs", "atom_counts", "labels", "grads", "ready")

    def wait(self):
        """Makes the current stream wait for the copies and the sort of this batch."""
        import torch
        cur = torch.cuda.current_stream()
        cur.wait_event(self.ready)
        for name in ("xs", "ys", "zs", "atom_types", "mol_idxs", "mol_atom_counts", "mol_offsets", "scatter_idxs",
                     "gather_idxs", "atom_counts", "grads"):
            t = getattr(self, name)
            if t is not None:
                t.record_stream(cur)       # the memory was allocated on the feeder's stream
        return self


class DeviceFeeder:
    """Iterates a RawDataset as DeviceBatch objects, one batch ahead of the consumer.

    Pinned staging buffers are allocated once (for the largest batch seen so far, two sets), copies run on
    a side stream of default priority, and `mol_offsets` + `ani_sort` are enqueued behind them on the same
    stream.  The consumer calls `batch.wait()` before using the tensors on its own stream."""

    def __init__(self, dataset, batch_size, shuffle=False, fuzz=None, dtype=np.float32, device="cuda:0", rng=None):
        import torch
        self.dataset, self.batch_size, self.shuffle, self.fuzz = dataset, batch_size, shuffle, fuzz
        self.dtype, self.device, self.rng = dtype, torch.device(device), rng
        self.stream = torch.cuda.Stream(device=self.device)
        self._pinned = [None, None]
        self._events = [None, None]       # consumer-side "done with this staging set" is implied by the H2D event

    def _staging(self, slot, n_atoms):
        import torch
        cur = self._pinned[slot]
        if cur is None or cur["cap"] < n_atoms:
            cap = max(n_atoms, 1024)
            tdt = torch.float32 if self.dtype == np.float32 else torch.float64
            cur = {"cap": cap,
                   "xyz": torch.empty((3, cap), dtype=tdt, pin_memory=True),
                   "ints": torch.empty((2, cap), dtype=torch.int32, pin_memory=True)}
            self._pinned[slot] = cur
        return cur

    def _enqueue(self, slot, item):
        import torch
        from . import ops
        mol_Xs, mol_ids, mol_yts, mol_grads = item
        xs, ys, zs, types, mids = split_columns(mol_Xs, mol_ids, self.dtype)
        n = xs.size
        n_mols = int(mids[-1]) + 1 if n else 0
        st = self._staging(slot, n)
        if self._events[slot] is not None:
            self._events[slot].synchronize()          # the previous copy out of this staging set has finished
        st["xyz"][0, :n] = torch.from_numpy(xs)
        st["xyz"][1, :n] = torch.from_numpy(ys)
        st["xyz"][2, :n] = torch.from_numpy(zs)
        st["ints"][0, :n] = torch.from_numpy(types)
        st["ints"][1, :n] = torch.from_numpy(mids)
        b = DeviceBatch()
        with torch.cuda.stream(self.stream):
            # each row of the staging arrays is contiguous pinned memory: five asynchronous copies
            b.xs, b.ys, b.zs = (st["xyz"][k, :n].to(self.device, non_blocking=True) for k in range(3))
            b.atom_types, b.mol_idxs = (st["ints"][k, :n].to(self.device, non_blocking=True) for k in range(2))
            copied = torch.cuda.Event()
            copied.record(self.stream)
            self._events[slot] = copied
            b.n_mols = n_mols
            b.mol_atom_counts, b.mol_offsets = ops.mol_offsets(b.mol_idxs, n_mols)
            b.scatter_idxs, b.gather_idxs, b.atom_counts = ops.ani_sort(b.atom_types)
            b.labels = mol_yts
            b.grads = None
            if mol_grads is not None:
                b.grads = torch.from_numpy(np.ascontiguousarray(mol_grads, dtype=self.dtype)).to(self.device)
            b.ready = torch.cuda.Event()
            b.ready.record(self.stream)
        return b

    def __iter__(self):
        it = self.dataset.iterate(self.batch_size, self.shuffle, self.fuzz, self.rng)
        slot, ahead = 0, None
        for item in it:
            nxt = self._enqueue(slot, item)
            slot ^= 1
            if ahead is not None:
                yield ahead
            ahead = nxt
        if ahead is not None:
            yield ahead
