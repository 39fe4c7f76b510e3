"""Pooled-lookup problems shaped like the reference's operator test
(cust_op/test/split_embedding_codegen_lookup_adagrad_function_test/torch/test_split_embedding_codegen_lookup_function.py):
several features may read one table (feature_map), bags of fixed or random length, and the unique inputs are built as
its generate_unique builds them (:268-287): per table torch.unique over the concatenated values of its features, the
start of the table's slice repeated once per feature."""
import numpy as np


class TbeProblem:
    def __init__(self, seed, tables, feature_map, batch, max_len, fixed_len=None, same_dim=False):
        """tables: [(rows, dim)], feature_map[f] = table of feature f (non-decreasing)."""
        rng = np.random.default_rng(seed)
        self.tables = tables
        self.feature_map = list(feature_map)
        self.F = len(feature_map)
        self.B = batch
        dims = [tables[t][1] for t in feature_map]
        self.d_offsets = np.concatenate([[0], np.cumsum(dims)]).astype(np.int32)
        self.total_d = int(self.d_offsets[-1])
        self.max_d = max(dims)
        sizes = [r * d for r, d in tables]
        table_w_off = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
        table_row_off = np.concatenate([[0], np.cumsum([r for r, _ in tables])]).astype(np.int64)
        self.table_w_off = table_w_off
        self.weights_offsets = np.array([table_w_off[t] for t in feature_map], dtype=np.int64)
        # one entry per feature, features of one table carry the table's start; the last entry is the total
        self.hash_size_cumsum = np.array([table_row_off[t] for t in feature_map] + [table_row_off[-1]], dtype=np.int64)
        if fixed_len is not None:
            lengths = np.repeat(np.asarray(fixed_len, dtype=np.int64), batch)
        else:
            lengths = rng.integers(0, max_len + 1, self.F * batch)
        self.lengths = lengths
        self.offsets = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int64)
        per_feature = []
        for f, t in enumerate(feature_map):
            n = int(lengths[f * batch:(f + 1) * batch].sum())
            per_feature.append(rng.integers(0, tables[t][0], n).astype(np.int64))
        self.per_feature = per_feature
        self.indices = np.concatenate(per_feature + [np.zeros(0, np.int64)])
        self.nnz = self.indices.size
        self.weights = rng.normal(0, 0.1, int(table_w_off[-1])).astype(np.float32)
        self.rng = rng

    def unique_inputs(self, indices=None):
        """(unique_ids, unique_offsets[F+1], unique_inverse[nnz]) as the reference's generate_unique makes them."""
        per_feature = self.per_feature
        if indices is not None:
            per_feature = [indices[self.offsets[f * self.B]:self.offsets[(f + 1) * self.B]] for f in range(self.F)]
        ids, inv, off = [], [], []
        start = 0
        seen = []
        for t in self.feature_map:
            if t not in seen:
                seen.append(t)
        for t in seen:
            feats = [f for f, tt in enumerate(self.feature_map) if tt == t]
            vals = np.concatenate([per_feature[f] for f in feats] + [np.zeros(0, np.int64)])
            u, i = np.unique(vals, return_inverse=True)
            ids.append(u)
            inv.append(i.astype(np.int64))
            off.extend(len(feats) * [start])
            start += u.size
        off.append(start)
        return (np.concatenate(ids + [np.zeros(0, np.int64)]).astype(np.int64), np.asarray(off, dtype=np.int64),
                np.concatenate(inv + [np.zeros(0, np.int64)]).astype(np.int64))

    def table_view(self, flat, t):
        r, d = self.tables[t]
        return flat[self.table_w_off[t]:self.table_w_off[t] + r * d].reshape(r, d)

    def grad_shape(self, pooling_mode):
        return (self.nnz, self.max_d) if pooling_mode == 2 else (self.B, self.total_d)
