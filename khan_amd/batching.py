"""Host batch assembly and device feeding for the featurizer.

`RawDataset` mirrors khan/data/dataset.py:7-183: molecules are ragged arrays of rows (type, x, y, z), a
batch is their concatenation plus, per atom, the index of its molecule inside the batch; the last
batch is not padded (dataset.py:118-183).

`PackedDataset` holds the same data packed once into flat arrays and assembles a batch with a native,
multi-threaded gather (csrc/host_batch.c) instead of one numpy operation per molecule.

`DeviceFeeder` is what the reference does with a feed dict and a staging queue
(khan/training/trainer_multi_tower.py:767-792, 291-303), done for one GPU with PyTorch as the memory
and stream plumbing: it splits a batch into the flat arrays the ops take (xs, ys, zs, atom types,
molecule indices), copies them through pinned host buffers with asynchronous host-to-device copies on a
side stream, runs `mol_offsets` and `ani_sort` on the device, and keeps one batch in flight while the
caller works on the previous one.
"""
import ctypes
import math
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
HOST_LIB_PATH = os.path.join(_HERE, "csrc", "libkhan_host.so")
_host_lib = None


def _host():
    """The native batch assembler (csrc/host_batch.c); no GPU code in it."""
    global _host_lib
    if _host_lib is None:
        if not os.path.exists(HOST_LIB_PATH):
            raise RuntimeError("%s is missing: run `python -m khan_amd.build`" % HOST_LIB_PATH)
        lib = ctypes.CDLL(HOST_LIB_PATH)
        vp, i64 = ctypes.c_void_p, ctypes.c_int64
        lib.khan_host_batch_offsets.restype = i64
        lib.khan_host_batch_offsets.argtypes = [vp, i64, vp, i64, vp]
        for name in ("khan_host_gather_f32", "khan_host_gather_f64"):
            fn = getattr(lib, name)
            fn.restype = None
            fn.argtypes = [vp, vp, vp, vp, vp, vp, i64, vp, vp, vp, vp, vp, vp, ctypes.c_int]
        lib.khan_host_gather_rows3_f64.restype = None
        lib.khan_host_gather_rows3_f64.argtypes = [vp, vp, vp, i64, vp, vp, ctypes.c_int]
        _host_lib = lib
    return _host_lib


def _np_ptr(a):
    return ctypes.c_void_p(a.ctypes.data)


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


class PackedDataset:
    """The same data set packed once into flat arrays: every atom's type and coordinates end to end plus the
    molecule offsets.  A batch is then gathered by a native routine (parallel over molecules) straight into the
    flat arrays the ops take, instead of one numpy operation per molecule; `iterate` still yields the
    reference's tuples.  Coordinates are kept in `dtype`, the precision the featurizer will run in."""

    def __init__(self, all_Xs, all_ys=None, all_grads=None, dtype=np.float32, n_threads=None):
        counts = np.array([len(m) for m in all_Xs], dtype=np.int64)
        self.offsets = np.zeros(len(counts) + 1, dtype=np.int64)
        np.cumsum(counts, out=self.offsets[1:])
        flat = np.concatenate([np.asarray(m, dtype=np.float64).reshape(-1, 4) for m in all_Xs], axis=0) \
            if len(counts) else np.zeros((0, 4))
        self.dtype = np.dtype(dtype)
        self.types = np.ascontiguousarray(flat[:, 0]).astype(np.int32)
        self.x, self.y, self.z = (np.ascontiguousarray(flat[:, k], dtype=self.dtype) for k in (1, 2, 3))
        self.ys = None if all_ys is None else np.asarray(all_ys)
        if self.ys is not None and len(self.ys) != len(counts):
            raise ValueError("all_ys must have one entry per molecule")
        self.grads = None
        if all_grads is not None:
            if len(all_grads) != len(counts):
                raise ValueError("all_grads must have one entry per molecule")
            self.grads = np.ascontiguousarray(np.concatenate([np.asarray(g, dtype=np.float64).reshape(-1, 3)
                                                              for g in all_grads], axis=0)) if len(counts) else np.zeros((0, 3))
        self.n_threads = int(n_threads) if n_threads else min(16, os.cpu_count() or 1)

    @classmethod
    def from_raw(cls, raw, dtype=np.float32, n_threads=None):
        return cls(raw.all_Xs, raw.all_ys, raw.all_grads, dtype, n_threads)

    def num_mols(self):
        return self.offsets.size - 1

    def num_batches(self, batch_size):
        return math.ceil(self.num_mols() / batch_size)

    def batch_atoms(self, sel):
        """-> (per-molecule offsets inside the batch [len(sel) + 1], number of atoms) for molecules `sel`."""
        sel = np.ascontiguousarray(sel, dtype=np.int64)
        out_off = np.empty(sel.size + 1, dtype=np.int64)
        n = _host().khan_host_batch_offsets(_np_ptr(self.offsets), self.num_mols(), _np_ptr(sel), sel.size, _np_ptr(out_off))
        if n < 0:
            raise IndexError("molecule index out of range")
        return sel, out_off, int(n)

    def gather_into(self, sel, out_off, xs, ys, zs, types, mol_ids):
        """Fills the first out_off[-1] elements of the given flat arrays (numpy views, e.g. of pinned tensors)."""
        for a, dt in ((xs, self.dtype), (ys, self.dtype), (zs, self.dtype), (types, np.int32), (mol_ids, np.int32)):
            if a.dtype != dt or not a.flags["C_CONTIGUOUS"] or a.size < out_off[-1]:
                raise ValueError("destination arrays must be contiguous, of the data set's types, and large enough")
        fn = _host().khan_host_gather_f32 if self.dtype == np.float32 else _host().khan_host_gather_f64
        fn(_np_ptr(self.offsets), _np_ptr(self.types), _np_ptr(self.x), _np_ptr(self.y), _np_ptr(self.z), _np_ptr(sel),
           sel.size, _np_ptr(out_off), _np_ptr(xs), _np_ptr(ys), _np_ptr(zs), _np_ptr(types), _np_ptr(mol_ids), self.n_threads)

    def gather(self, sel):
        """-> (xs, ys, zs, atom types, molecule index per atom) of the batch made of molecules `sel`."""
        sel, out_off, n = self.batch_atoms(sel)
        xs, ys, zs = (np.empty(n, dtype=self.dtype) for _ in range(3))
        types, mol_ids = np.empty(n, dtype=np.int32), np.empty(n, dtype=np.int32)
        self.gather_into(sel, out_off, xs, ys, zs, types, mol_ids)
        return xs, ys, zs, types, mol_ids

    def gather_grads(self, sel, out_off):
        out = np.empty((int(out_off[-1]), 3), dtype=np.float64)
        _host().khan_host_gather_rows3_f64(_np_ptr(self.offsets), _np_ptr(self.grads), _np_ptr(sel), sel.size,
                                           _np_ptr(out_off), _np_ptr(out), self.n_threads)
        return out

    def selections(self, batch_size, shuffle, rng=None):
        """The molecule indices of every batch, in order (the last batch is not padded)."""
        rng = np.random.default_rng() if rng is None else rng
        perm = np.arange(self.num_mols(), dtype=np.int64)
        if shuffle:
            rng.shuffle(perm)
        for batch_idx in range(self.num_batches(batch_size)):
            yield perm[batch_idx * batch_size:min((batch_idx + 1) * batch_size, self.num_mols())]

    def iterate(self, batch_size, shuffle, fuzz=None, rng=None):
        """Same tuples as RawDataset.iterate: (mol_Xs [N,4] float64, mol_ids, mol_yts or None, mol_grads or None)."""
        rng = np.random.default_rng() if rng is None else rng
        for sel in self.selections(batch_size, shuffle, rng):
            sel, out_off, n = self.batch_atoms(sel)
            xs, ys, zs, types, mol_ids = self.gather(sel)
            mol_Xs = np.stack([types.astype(np.float64), xs.astype(np.float64), ys.astype(np.float64), zs.astype(np.float64)], axis=1)
            if fuzz is not None:
                mol_Xs[:, 1:4] += rng.uniform(-fuzz, fuzz, (n, 3))
            mol_yts = None if self.ys is None else list(self.ys[sel])
            mol_grads = None if self.grads is None else self.gather_grads(sel, out_off)
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
                 "scatter_idxs", "gather_idxs", "atom_counts", "size_order", "counts_pinned", "labels", "grads", "ready")

    def host_counts(self):
        """-> (atoms per type [4], the size order on the device, molecules per size class [4] on the host): what the
        host has to know before it can launch the passes.  One 32-byte copy, enqueued by the feeder behind the
        sort; this waits for it."""
        self.ready.synchronize()
        return self.counts_pinned[0:4].tolist(), self.size_order, self.counts_pinned[4:8].clone()

    @classmethod
    def from_device_arrays(cls, xs, ys, zs, atom_types, mol_idxs, n_mols):
        """A batch from arrays that are on the GPU already: runs `mol_offsets`, `ani_sort` and `size_order` on the
        current stream and enqueues the copy of the counts."""
        import torch
        from . import ops
        b = cls()
        b.xs, b.ys, b.zs, b.atom_types, b.mol_idxs, b.n_mols = xs, ys, zs, atom_types, mol_idxs, n_mols
        b.labels = b.grads = None
        b.finish_on_current_stream()
        return b

    def finish_on_current_stream(self):
        """Offsets, type sort, size order and the copy of the counts for the arrays already in place; records `ready`."""
        import torch
        from . import ops
        self.mol_atom_counts, self.mol_offsets = ops.mol_offsets(self.mol_idxs, self.n_mols)
        self.scatter_idxs, self.gather_idxs, self.atom_counts = ops.ani_sort(self.atom_types)
        self.size_order = ops.size_order(self.mol_atom_counts)
        self.counts_pinned = torch.empty(8, dtype=torch.int32, pin_memory=True)     # from the pinned-memory cache
        self.counts_pinned[0:4].copy_(self.atom_counts, non_blocking=True)
        self.counts_pinned[4:8].copy_(self.size_order[-4:], non_blocking=True)
        self.ready = torch.cuda.Event()
        self.ready.record()

    def wait(self):
        """Makes the current stream wait for the copies and the sort of this batch."""
        import torch
        cur = torch.cuda.current_stream()
        cur.wait_event(self.ready)
        for name in ("xs", "ys", "zs", "atom_types", "mol_idxs", "mol_atom_counts", "mol_offsets", "scatter_idxs",
                     "gather_idxs", "atom_counts", "size_order", "grads"):
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

    def _fill_from_tuple(self, slot, item):
        """Reference-style tuple -> staging set; returns (n atoms, n molecules, labels, gradients)."""
        import torch
        mol_Xs, mol_ids, mol_yts, mol_grads = item
        xs, ys, zs, types, mids = split_columns(mol_Xs, mol_ids, self.dtype)
        n = xs.size
        # one molecule per label: trailing molecules without atoms still count (mol_ids alone would drop them)
        n_mols = len(mol_yts) if mol_yts is not None else (int(mids[-1]) + 1 if n else 0)
        if n and int(mids[-1]) >= n_mols:
            raise ValueError("mol_ids names molecule %d but the batch has %d labels" % (int(mids[-1]), n_mols))
        st = self._staging(slot, n)
        if self._events[slot] is not None:
            self._events[slot].synchronize()          # the previous copy out of this staging set has finished
        st["xyz"][0, :n] = torch.from_numpy(xs)
        st["xyz"][1, :n] = torch.from_numpy(ys)
        st["xyz"][2, :n] = torch.from_numpy(zs)
        st["ints"][0, :n] = torch.from_numpy(types)
        st["ints"][1, :n] = torch.from_numpy(mids)
        return n, n_mols, mol_yts, mol_grads

    def _fill_from_packed(self, slot, sel):
        """Molecule selection of a PackedDataset -> staging set, gathered natively into the pinned buffers."""
        ds = self.dataset
        sel, out_off, n = ds.batch_atoms(sel)
        st = self._staging(slot, n)
        if self._events[slot] is not None:
            self._events[slot].synchronize()
        xyz, ints = st["xyz"].numpy(), st["ints"].numpy()
        ds.gather_into(sel, out_off, xyz[0], xyz[1], xyz[2], ints[0], ints[1])
        if self.fuzz is not None:
            rng = np.random.default_rng() if self.rng is None else self.rng
            xyz[:, :n] += rng.uniform(-self.fuzz, self.fuzz, (3, n)).astype(xyz.dtype)
        labels = None if ds.ys is None else ds.ys[sel]            # an array here (a list from a RawDataset)
        grads = None if ds.grads is None else ds.gather_grads(sel, out_off)
        return n, sel.size, labels, grads

    def _enqueue(self, slot, item):
        import torch
        from . import ops
        if isinstance(self.dataset, PackedDataset):
            n, n_mols, mol_yts, mol_grads = self._fill_from_packed(slot, item)
        else:
            n, n_mols, mol_yts, mol_grads = self._fill_from_tuple(slot, item)
        st = self._pinned[slot]
        b = DeviceBatch()
        with torch.cuda.stream(self.stream):
            # each row of the staging arrays is contiguous pinned memory: five asynchronous copies
            b.xs, b.ys, b.zs = (st["xyz"][k, :n].to(self.device, non_blocking=True) for k in range(3))
            b.atom_types, b.mol_idxs = (st["ints"][k, :n].to(self.device, non_blocking=True) for k in range(2))
            copied = torch.cuda.Event()
            copied.record(self.stream)
            self._events[slot] = copied
            b.n_mols = n_mols
            b.labels = mol_yts
            b.grads = None
            if mol_grads is not None:
                b.grads = torch.from_numpy(np.ascontiguousarray(mol_grads, dtype=self.dtype)).to(self.device)
            b.finish_on_current_stream()          # the feeder's stream is current here
        return b

    def __iter__(self):
        if isinstance(self.dataset, PackedDataset):
            if self.dataset.dtype != np.dtype(self.dtype):
                raise TypeError("the packed data set holds %s coordinates, the feeder was asked for %s"
                                % (self.dataset.dtype, np.dtype(self.dtype)))
            it = self.dataset.selections(self.batch_size, self.shuffle, self.rng)
        else:
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
