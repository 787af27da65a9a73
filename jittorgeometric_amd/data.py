"""Graph containers with the attribute names of the reference
(jittor_geometric/data/data.py:42-52).  The arrays are torch tensors:
int32 indices/offsets, float32 weights."""


class CSR:
    def __init__(self, column_indices=None, row_offset=None, edge_weight=None):
        self.column_indices = column_indices
        self.row_offset = row_offset
        self.edge_weight = edge_weight


class CSC:
    def __init__(self, row_indices=None, column_offset=None, edge_weight=None):
        self.row_indices = row_indices
        self.column_offset = column_offset
        self.edge_weight = edge_weight
