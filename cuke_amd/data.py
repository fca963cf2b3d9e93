"""Dataset reader and batch sampler for the KGE path (the steps in front of the score kernels).

Mirrors the reference's data layer where it can be mirrored offline:
``KGDataset`` reads the same five-file layout as apps/kge/data/preprocess.py:26-99 (``id\\tname``
dictionaries, ``head\\trel\\ttail`` triples; it does not download anything), and ``TrainSampler``
plays the role of ``TrainDataset.create_sampler`` (apps/kge/data/sampler.py:304-353): batches of
positives plus, per chunk of ``neg_chunk_size`` positives, ``neg_sample_size`` shared negative
entities drawn uniformly (exclude_positive=False) -- drawn on the GPU by ``kge_sample_negatives``.
The negatives replace the tail, the head, or alternate between the two from batch to batch, as the
reference's head / tail samplers do (apps/kge/data/sampler.py:287-353, 451-487).
"""
from __future__ import annotations

import ctypes as C

import numpy as np
import torch

from . import _lib


class KGDataset:
    """entities / relations dictionaries (``id<delim>name``) and train / valid / test triples
    (``head<delim>rel<delim>tail`` by name; ``format`` gives the column order)."""

    def __init__(self, entity_path, relation_path, train_path, valid_path=None, test_path=None,
                 format=(0, 1, 2), delimiter="\t", skip_first_line=False):
        self.delimiter = delimiter
        self.entity2id, self.n_entities = self._read_dict(entity_path)
        self.relation2id, self.n_relations = self._read_dict(relation_path)
        self.train = self.read_triple(train_path, skip_first_line, format)
        self.valid = self.read_triple(valid_path, skip_first_line, format)
        self.test = self.read_triple(test_path, skip_first_line, format)

    def _read_dict(self, path):
        mapping = {}
        with open(path) as f:
            for line in f:
                line = line.rstrip("\n")
                if not line:
                    continue
                idx, name = line.split(self.delimiter)
                mapping[name] = int(idx)
        return mapping, len(mapping)

    def read_triple(self, path, skip_first_line=False, format=(0, 1, 2)):
        if path is None:
            return None
        cols = ([], [], [])
        with open(path) as f:
            if skip_first_line:
                f.readline()
            for line in f:
                parts = line.rstrip("\n").split(self.delimiter)
                if len(parts) < 3:
                    continue
                cols[0].append(self.entity2id[parts[format[0]]])
                cols[1].append(self.relation2id[parts[format[1]]])
                cols[2].append(self.entity2id[parts[format[2]]])
        heads, rels, tails = (np.asarray(c, dtype=np.int64) for c in cols)
        return heads, rels, tails


class TrainSampler:
    """Iterates over (h, r, t, neg) device tensors: ``batch_size`` positives (a seeded shuffle of the
    training triples, reshuffled every epoch) and ``neg_sample_size`` shared negative entities for
    every chunk of ``neg_chunk_size`` positives.

    ``mode`` says which side the negatives replace: ``'tail'``, ``'head'``, or ``'both'``, which
    alternates like the reference's NewBidirectionalOneShotIterator (apps/kge/data/sampler.py:481-487:
    first batch tail, second head, ...).  ``neg_mode`` holds the mode of the batch returned last; pass
    it to ``KGEModel.score(..., neg_mode=sampler.neg_mode)``."""

    def __init__(self, triples, n_entities, batch_size, neg_sample_size, neg_chunk_size=None, shuffle=True,
                 seed=0, device="cuda:0", mode="tail"):
        if mode not in ("tail", "head", "both"):
            raise ValueError("mode is 'tail', 'head' or 'both'")
        self.mode = mode
        self.neg_mode = "head" if mode == "head" else "tail"
        self.h, self.r, self.t = (np.asarray(x, dtype=np.int64) for x in triples)
        self.n_entities, self.batch = int(n_entities), int(batch_size)
        self.n_neg = int(neg_sample_size)
        self.chunk = int(neg_chunk_size) if neg_chunk_size else self.n_neg
        if self.batch % self.chunk:
            raise ValueError("batch_size must be a multiple of neg_chunk_size")
        if len(self.h) < self.batch:
            raise ValueError("fewer training triples than one batch")
        self.shuffle, self.seed = shuffle, int(seed)
        self.dev = torch.device(device)
        self.step = 0
        self._order, self._pos, self._epoch = None, 0, 0

    def _next_ids(self):
        if self._order is None or self._pos + self.batch > len(self._order):
            n = len(self.h)
            self._order = np.random.default_rng([self.seed, self._epoch]).permutation(n) if self.shuffle \
                else np.arange(n)
            self._pos, self._epoch = 0, self._epoch + 1
        ids = self._order[self._pos:self._pos + self.batch]
        self._pos += self.batch
        return ids

    def __iter__(self):
        return self

    def __next__(self):
        ids = self._next_ids()
        h, r, t = (torch.from_numpy(x[ids]).to(self.dev) for x in (self.h, self.r, self.t))
        count = (self.batch // self.chunk) * self.n_neg
        neg = torch.empty(count, dtype=torch.int64, device=self.dev)
        _lib.check(_lib.lib().kge_sample_negatives(C.c_void_p(neg.data_ptr()), count, self.n_entities,
                                                   self.seed, self.step,
                                                   C.c_void_p(torch.cuda.current_stream().cuda_stream)),
                   "kge_sample_negatives")
        if self.mode == "both":
            self.neg_mode = "head" if self.step % 2 else "tail"
        self.step += 1
        return h, r, t, neg
