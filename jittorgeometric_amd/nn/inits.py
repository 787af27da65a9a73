"""Parameter initialisers of the reference (nn/inits.py:19-22,59-61)."""
import math

import torch


def glorot(t):
    if t is not None:
        stdv = math.sqrt(6.0 / (t.size(-2) + t.size(-1)))
        with torch.no_grad():
            t.uniform_(-stdv, stdv)


def zeros(t):
    if t is not None:
        with torch.no_grad():
            t.zero_()
