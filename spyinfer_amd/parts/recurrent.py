"""Gated recurrences with a state of fixed size per request.

``MinGRU``: the gates read only the current token, so all of a step's gates come from one product and the
recurrence itself is a scan over the tokens:  z = sigmoid(Wz h + bz), u = Wx h + bx, candidate c = u + 1/2 where
u >= 0 and sigmoid(u) where u < 0;  S_t = (1 - z) S_(t-1) + z c per channel;  output Wo (S_t * silu(Wg h)).  The state
starts at zero, is float32 and lives in the request's slot; everything behind the projections is float32.
"""
from __future__ import annotations

import numpy as np
import torch

from ..cache.spec import FixedState
from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Mixer

#: tokens of an entry that one thread walks in a row; longer entries are cut, so that a long portion has blocks for
#: the whole device (the pieces' effects on the state are composed, the recurrence being linear in it)
SCAN_PIECE = 32


def plan_scan_pieces(batch, piece: int = SCAN_PIECE) -> None:
    """Adds the step's entries cut into pieces of at most ``piece`` tokens: int32 [4 n] = entry, first row, end row,
    index of the entry's first piece.  Once per step."""
    if "scan_pieces" in batch.shared:
        return
    lens = batch.lens.astype(np.int64)
    cu = batch.host_array("cu_q").astype(np.int64)
    counts = (lens + piece - 1) // piece
    first = np.zeros(batch.S + 1, dtype=np.int64)
    np.cumsum(counts, out=first[1:])
    n = int(first[-1])
    entry = np.repeat(np.arange(batch.S, dtype=np.int64), counts)
    k = np.arange(n, dtype=np.int64) - first[:-1][entry]
    t0 = cu[:-1][entry] + k * piece
    t1 = np.minimum(t0 + piece, cu[1:][entry])
    batch.add_array("scan_pieces", np.concatenate([entry, t0, t1, first[:-1][entry]]).astype(np.int32))
    batch.shared["scan_pieces"] = (n, bool((counts > 1).any()))


class MinGRU(Mixer):
    def __init__(self, hidden_size: int, width: int, names=("z", "z.b", "x", "x.b", "g", "o")):
        self.hidden_size, self.width, self.names = hidden_size, width, names
        self.w_zxg = self.w_zxg_tiled = self.w_o = self.w_o_tiled = self.b_z = self.b_x = None

    def weight_specs(self, prefix):
        H, W = self.hidden_size, self.width
        z, zb, x, xb, g, o = (prefix + "." + n for n in self.names)
        return [WeightSpec(z, (W, H)), WeightSpec(zb, (W,), "bias"), WeightSpec(x, (W, H)), WeightSpec(xb, (W,), "bias"),
                WeightSpec(g, (W, H)), WeightSpec(o, (H, W))]

    def bind(self, prefix, weights):
        z, zb, x, xb, g, o = (prefix + "." + n for n in self.names)
        mats = [weights.pop(n) for n in (z, x, g)]
        if len({m.dtype for m in mats}) > 1:
            mats = [m.float() for m in mats]
        # one product for the three projections: rows [z | x | g]
        self.w_zxg, self.w_zxg_tiled = ops.weight_forms(torch.cat(mats, dim=0).contiguous())
        del mats
        self.w_o, self.w_o_tiled = ops.weight_forms(weights.pop(o))
        self.b_z, self.b_x = weights[zb], weights[xb]
        if self.b_z.dtype != self.b_x.dtype:
            self.b_z, self.b_x = self.b_z.float(), self.b_x.float()

    def cache_spec(self):
        return FixedState((self.width,), "float32")

    def plan(self, batch) -> None:
        plan_scan_pieces(batch)

    def plan_arrays(self, entries):
        return {"scan_pieces": 4 * entries}

    def capturable(self, batch):
        return True

    def forward(self, x, batch, cache, store=True):
        if not store:
            raise ValueError("a recurrence cannot run on another layer's state without writing it")
        zxg = ops.linear_few(x, self.w_zxg, self.w_zxg_tiled)
        n, multi = batch.shared["scan_pieces"]
        y = ops.mingru(zxg, self.b_z, self.b_x, cache.state, batch.array("scan_pieces"), n, multi, batch.array("slot_ids"))
        return ops.linear_few(y, self.w_o, self.w_o_tiled)
