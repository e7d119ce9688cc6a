"""GPTQ weight quantisation in the Hadamard-rotated basis (reference: flh/nn/gptq.py).

The reference's calibration flow (flh/quantized_model/modeling_llama.py:810-836): a float nn.Linear, `add_batch` for
every calibration input of the layer, `fasterquant`, which replaces `layer.weight` by the DEQUANTISED weights of the
rotated basis, then `LinearFLH.from_float(layer, no_hadamard=True)` packs them.  This module keeps those names and
arguments.  The arithmetic is GPTQ's: with H = 2/n sum x x^T over the (rotated) calibration inputs and the columns
taken left to right (or by decreasing diag(H) with `actorder`), column i is rounded to its group's grid and the error,
divided by the i-th diagonal entry of the upper Cholesky factor of H^-1, is pushed onto the columns that follow along
that factor's row -- evaluated block by block of `blocksize` columns, with the grid of every group fixed beforehand from
the rotated, clipped weights ("static groups", the only mode the reference's group path has).

Everything here is tensor arithmetic on the layer's device (float32, as the reference); the activation side of the path
does not enter.
"""
import math

import torch

from .quantization import fast_hadamard_transform


class GPTQQuantizer:
    """The grid of one weight slice (flh/nn/gptq.py:27-112): per group of `groupsize` columns when that divides the
    slice, else one scale per row."""

    def __init__(self, bits, groupsize=-1, sym=True, clip_ratio=1.0):
        self.bits, self.groupsize, self.sym, self.clip_ratio = bits, groupsize, sym, clip_ratio
        self.maxq = 2 ** (bits - 1) - 1 if sym else 2 ** bits - 1
        self.scale = None
        self.zero = None

    def ready(self):
        return self.scale is not None and bool(torch.all(self.scale != 0))

    def _grouped(self, W):
        return self.groupsize > 0 and W.shape[1] % self.groupsize == 0

    def _clip_weight(self, W):
        if self.clip_ratio >= 1.0:
            return W
        if self._grouped(W):
            g = W.view(W.shape[0], -1, self.groupsize)
            bound = g.abs().amax(dim=2, keepdim=True) * self.clip_ratio
            return torch.clamp(g, -bound, bound).view(W.shape)
        bound = W.abs().amax(dim=1, keepdim=True) * self.clip_ratio
        return torch.clamp(W, -bound, bound)

    def find_params(self, W, weight=True):
        W = self._clip_weight(W.float())
        if self.bits >= 16:
            return
        rows = W.shape[0]
        v = W.view(rows, -1, self.groupsize) if self._grouped(W) else W.view(rows, 1, -1)
        if self.sym:
            self.scale = (v.abs().amax(dim=2).clamp(min=1e-5) / self.maxq)
            self.zero = torch.zeros_like(self.scale)
        else:
            hi, lo = v.amax(dim=2), v.amin(dim=2)
            flat = (hi == 0) & (lo == 0)
            hi, lo = torch.where(flat, torch.ones_like(hi), hi), torch.where(flat, -torch.ones_like(lo), lo)
            self.scale = ((hi - lo) / self.maxq).clamp(min=1e-5)
            self.zero = torch.round(-lo / self.scale)
        if not self._grouped(W):          # one scale per row, repeated over the columns as the reference stores it
            self.scale = self.scale.repeat(1, W.shape[1])
            self.zero = self.zero.repeat(1, W.shape[1])

    def quantize(self, w, col=0):
        """One column `w` [rows] onto the grid: scale column `col` when there is one, else column 0."""
        if not self.ready():
            return w
        pick = col if (self.scale.dim() > 1 and col < self.scale.shape[1]) else 0
        scale = (self.scale if self.scale.dim() == 1 else self.scale[:, pick]).to(w.device)
        if self.clip_ratio < 1.0:
            bound = scale * self.maxq * self.clip_ratio
            w = torch.clamp(w, -bound, bound)
        if self.sym:
            return scale * torch.clamp(torch.round(w / scale), -(self.maxq + 1), self.maxq)
        zero = self.zero[:, pick].to(w.device)
        return scale * (torch.clamp(torch.round(w / scale + zero), 0, self.maxq) - zero)


class FLHGPTQ:
    def __init__(self, layer, dual_hadamard=False):
        self.layer = layer
        self.dual_hadamard = dual_hadamard
        self.dev = layer.weight.device
        self.rows, self.columns = layer.weight.shape
        self.H = torch.zeros((self.columns, self.columns), device=self.dev, dtype=torch.float32)
        self.nsamples = 0
        self.out_list = []

    def add_batch(self, inp, out, group_size=-1):
        """Running mean of 2 x x^T over the rotated inputs (flh/nn/gptq.py:127-144): inp [..., columns]."""
        rows = inp.reshape(-1, inp.shape[-1])
        n = rows.shape[0]
        rows = fast_hadamard_transform(rows.float(), group_size=group_size if group_size > 0 else None)
        self.H *= self.nsamples / (self.nsamples + n)
        self.nsamples += n
        x = math.sqrt(2 / self.nsamples) * rows.t()
        self.H += x.matmul(x.t())
        if out is not None:
            self.out_list.append(out.reshape(-1, out.shape[-1]))

    def fasterquant(self, group_size=128, blocksize=128, percdamp=0.01, actorder=False, sym=True, bits=4,
                    dual_hadamard=None, clip_ratio=1.0):
        if dual_hadamard is None:
            dual_hadamard = self.dual_hadamard
        group_size = group_size if group_size > 0 and self.columns % group_size == 0 else -1
        gs = group_size if group_size > 0 else None
        W = fast_hadamard_transform(self.layer.weight.data.clone().float(), group_size=gs)
        if dual_hadamard:
            W = fast_hadamard_transform(W.T, group_size=gs).T
        self.quantizer = GPTQQuantizer(bits=bits, groupsize=group_size, sym=sym, clip_ratio=clip_ratio)

        H = self.H
        del self.H
        dead = torch.diag(H) == 0
        H[dead, dead] = 1
        W[:, dead] = 0
        if clip_ratio < 1.0:
            W = self.quantizer._clip_weight(W)
        # the grid of every column, fixed before any error is pushed around: per group, or one per row
        grids = []
        if group_size > 0:
            for start in range(0, self.columns, group_size):
                q = GPTQQuantizer(bits=bits, groupsize=group_size, sym=sym, clip_ratio=clip_ratio)
                q.find_params(W[:, start:start + group_size])
                grids.append(q)
        else:
            self.quantizer.find_params(W)

        order = torch.arange(self.columns, device=self.dev)
        if actorder:
            order = torch.argsort(torch.diag(H), descending=True)
            W = W[:, order]
            H = H[order][:, order]
        idx = torch.arange(self.columns, device=self.dev)
        H[idx, idx] += percdamp * torch.mean(torch.diag(H))
        # upper Cholesky factor of H^-1: row i carries what column i's error does to the columns after it
        U = torch.linalg.cholesky(torch.cholesky_inverse(torch.linalg.cholesky(H)), upper=True)
        source = order.tolist()                         # original column of each processed position

        Q = torch.zeros_like(W)
        for b0 in range(0, self.columns, blocksize):
            b1 = min(b0 + blocksize, self.columns)
            Wb = W[:, b0:b1].clone()
            Eb = torch.zeros_like(Wb)
            Ub = U[b0:b1, b0:b1]
            for i in range(b1 - b0):
                w = Wb[:, i]
                grid = grids[source[b0 + i] // group_size] if group_size > 0 else self.quantizer
                q = grid.quantize(w, 0)
                Q[:, b0 + i] = q
                e = (w - q) / Ub[i, i]
                Wb[:, i:] -= e.unsqueeze(1) * Ub[i, i:].unsqueeze(0)
                Eb[:, i] = e
            W[:, b1:] -= Eb.matmul(U[b0:b1, b1:])
        if actorder:
            Q = Q[:, torch.argsort(order)]
        self.layer.weight.data = Q.to(self.layer.weight.dtype).reshape(self.layer.weight.shape)

    def free(self):
        self.H = None
        if torch.cuda.is_available():
            torch.cuda.empty_cache()
