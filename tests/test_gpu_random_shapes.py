"""Seeded sweep over random shapes: forest / fern operators (stateless, from walk records, both backward modes, subsets
of the gradients), the convolutional operators in 1 to 3 dimensions, and the forest that stores its result as an image
with the backward that reads the image gradient -- each case against the CPU oracle: forward bit for bit; gradients
within 1e-5 (float32) / 1e-12 (float64) of the oracle in the data's precision plus that serial loop's own distance
from its float64 evaluation, and within the same tolerance, with no slack, of the float64 evaluation itself (the sweep
reaches shapes with tens of thousands of terms per threshold). The shapes come from a fixed seed, so the
sweep is the same on every run; sizes are bounded so that the oracle finishes the whole sweep in well under a minute."""
import random

import pytest
import torch

from conftest import make_conv, make_forest, rel_err
from oracle import hinge_oracle as ho
import hingetree_cpp as ops

pytestmark = pytest.mark.gpu

SEED, CASES = 11, 40


class _Sweep:
    def __init__(self, dev):
        self.dev = dev
        self.rng = random.Random(SEED)
        self.failures = []

    def report(self, tag, ok, info):
        if not ok:
            self.failures.append((tag, info))

    def forest_case(self, i):
        fern = self.rng.random() < 0.5
        dtype = torch.float32 if self.rng.random() < 0.75 else torch.float64
        D = self.rng.choice([1, 2, 3, 4, 5, 6, 7, 8, 10, 12])
        B = self.rng.choice([1, 2, 3, 17, 64, 65, 200, 1000, 3000])
        F = self.rng.choice([1, 2, 7, 16, 33, 100, 257, 1024, 1500])
        Kd = self.rng.choice([[], [], [], [1], [3], [2, 3], [65], [8, 9]])
        T = self.rng.choice([1, 2, 3, 8, 17, 64, 100, 257, 600])
        Md = self.rng.choice([[], [1], [2], [3], [4], [7], [10], [16], [17], [2, 2], [33], [70]])
        if (B * max(1, torch.tensor(Kd).prod().item() if Kd else 1)) * T * (2 ** D) > 4e8: return
        tag = f"forest#{i} B={B} F={F} K={Kd} T={T} D={D} M={Md} fern={fern} {dtype}"
        x, thr, ordn, w, gout = make_forest(B, F, Kd, T, D, Md, fern, dtype, seed=i)
        pre = 'fern_' if fern else 'tree_'
        g = [t.to(self.dev) for t in (x, thr, ordn, w, gout)]
        ref = ho.forward(x, thr, ordn, w, fern)
        self.report(tag + ' fwd', torch.equal(getattr(ops, pre + 'forward')(*g[:4]).cpu(), ref), '')
        out, rec = getattr(ops, pre + 'forward_records')(*g[:4])
        self.report(tag + ' fwd_rec', torch.equal(out.cpu(), ref), '')
        r = ho.backward(x, thr, ordn, w, gout, fern=fern)
        x64 = [t.double() if t.is_floating_point() else t for t in (x, thr, ordn, w, gout)]
        r64 = ho.backward(*x64, fern=fern)
        tol = 1e-5 if dtype == torch.float32 else 1e-12
        need = self.rng.choice([(True, True, True), (True, True, True), (True, False, False), (False, True, False), (False, False, True), (True, False, True)])
        for mode in ('backward', 'backward_deterministic'):
            d = getattr(ops, pre + mode)(g[0], need[0], g[1], need[1], g[2], False, g[3], need[2], g[4])
            for k, (got, want, w64) in enumerate(zip((d[0], d[1], d[3]), r, r64)):
                if not need[k]:
                    self.report(tag + f' {mode} none{k}', got is None, ''); continue
                slack = rel_err(want.double(), w64)
                e = rel_err(got.cpu(), want)
                self.report(tag + f' {mode} g{k}', e <= tol + slack and rel_err(got.cpu().double(), w64) <= tol, (e, slack))
        if rec is not None:
            for det in (False, True):
                d = getattr(ops, pre + 'backward_records')(rec, det, g[0], True, g[1], True, g[2], False, g[3], True, g[4])
                for k, (got, w64) in enumerate(zip((d[0], d[1], d[3]), r64)):
                    self.report(tag + f' rec det={det} g{k}', rel_err(got.cpu().double(), w64) <= tol, rel_err(got.cpu().double(), w64))
    def conv_case(self, i):
        nd = self.rng.choice([1, 2, 2, 3])
        fern = self.rng.random() < 0.5
        dtype = torch.float32 if self.rng.random() < 0.75 else torch.float64
        size = [self.rng.choice([5, 9, 16, 33, 40]) for _ in range(nd)]
        if nd == 3: size = [min(s, 12) for s in size]
        ker = [self.rng.choice([1, 2, 3]) for _ in range(nd)]
        st = [self.rng.choice([1, 1, 2]) for _ in range(nd)]
        pad = [self.rng.choice([0, 1, 2]) for _ in range(nd)]
        dil = [self.rng.choice([1, 1, 2]) for _ in range(nd)]
        B, C, Cout, D = self.rng.choice([1, 2, 5]), self.rng.choice([1, 3, 5, 16, 24, 40]), self.rng.choice([1, 4, 7, 70]), self.rng.choice([1, 2, 3, 5])
        Md = self.rng.choice([[], [], [3], [17]])
        ok_geo = all(s + 2 * p >= k + (k - 1) * (d - 1) for s, p, k, d in zip(size, pad, ker, dil))
        tag = f"conv#{i} nd={nd} B={B} C={C} Cout={Cout} size={size} D={D} M={Md} ker={ker} st={st} pad={pad} dil={dil} fern={fern} {dtype}"
        x, thr, ordn, w = make_conv(B, C, Cout, size, D, Md, ker, fern, dtype, seed=i)
        pre = ('fern_' if fern else 'tree_') + f'conv{nd}d_'
        g = [t.to(self.dev) for t in (x, thr, ordn, w)]
        if not ok_geo:
            try:
                getattr(ops, pre + 'forward')(*g, ker, st, pad, dil); self.report(tag, False, 'no error for bad geometry')
            except RuntimeError: pass
            return
        ref = ho.conv_forward(x, thr, ordn, w, ker, st, pad, dil, fern)
        out = getattr(ops, pre + 'forward')(*g, ker, st, pad, dil)
        self.report(tag + ' fwd', out.shape == ref.shape and torch.equal(out.cpu(), ref), '')
        if ref.numel() == 0: return
        gout = torch.randn(ref.shape, generator=torch.Generator().manual_seed(i), dtype=dtype)
        r = ho.conv_backward(x.double(), thr.double(), ordn, w.double(), gout.double(), ker, st, pad, dil, fern=fern)
        need = self.rng.choice([(True, True, True), (True, True, True), (True, True, False), (True, False, True), (True, False, False), (False, True, True)])
        d = getattr(ops, pre + 'backward')(g[0], need[0], g[1], need[1], g[2], False, g[3], need[2], gout.to(self.dev), ker, st, pad, dil)
        tol = 1e-5 if dtype == torch.float32 else 1e-12
        for k, (got, want) in enumerate(zip((d[0], d[1], d[3]), r)):
            if not need[k]:
                self.report(tag + f' bwd none{k}', got is None, ''); continue
            self.report(tag + f' bwd {need} g{k}', rel_err(got.cpu().double(), want) <= tol, rel_err(got.cpu().double(), want))
    def expanded_case(self, i):
        nd = self.rng.choice([2, 2, 3])
        fern = self.rng.random() < 0.5
        dtype = torch.float32 if self.rng.random() < 0.75 else torch.float64
        tiles = [self.rng.choice([1, 2, 3, 7, 12, 40]) for _ in range(nd)]
        if nd == 3: tiles = [min(t, 12) for t in tiles]
        window = [self.rng.choice([1, 2, 3, 4, 8]) for _ in range(nd)]
        padding = [self.rng.choice([0, 0, 1, 2, 4, 8]) for _ in range(nd)]
        B, F, T, D = self.rng.choice([1, 2, 9, 40]), self.rng.choice([1, 5, 30]), self.rng.choice([1, 3, 20, 100]), self.rng.choice([1, 2, 4, 6])
        if B * T * 2 ** D * torch.tensor(tiles).prod().item() * torch.tensor(window).prod().item() > 2e8: return
        size = [t * w - ((2 * p) // w) * w for t, w, p in zip(tiles, window, padding)]
        tag = f"expanded#{i} B={B} F={F} tiles={tiles} T={T} D={D} window={window} pad={padding} fern={fern} {dtype}"
        x, thr, ordn, w, _ = make_forest(B, F, tiles, T, D, window, fern, dtype, seed=i)
        pre = 'fern_' if fern else 'tree_'
        g = [t.to(self.dev) for t in (x, thr, ordn, w)]
        if any(n < 1 for n in size):
            try:
                getattr(ops, pre + 'forward_expanded')(*g, padding); self.report(tag, False, 'no error for empty image')
            except ValueError: pass
            return
        want = ho.expand(ho.forward(x, thr, ordn, w, fern), padding)
        got = getattr(ops, pre + 'forward_expanded')(*g, padding)
        self.report(tag, got.shape == want.shape and torch.equal(got.cpu(), want), '')
        gimg = torch.randn(want.shape, generator=torch.Generator().manual_seed(i + 5), dtype=dtype)
        gt = ho.contract(gimg, window, padding)
        x64 = [t.double() if t.is_floating_point() else t for t in (x, thr, ordn, w, gt)]
        r64 = ho.backward(*x64, fern=fern)
        tol = 1e-5 if dtype == torch.float32 else 1e-12
        for det in (False, True):
            d = getattr(ops, pre + 'backward_expanded')(det, padding, g[0], True, g[1], True, g[2], False, g[3], True, gimg.to(self.dev))
            for k, (gotg, w64) in enumerate(zip((d[0], d[1], d[3]), r64)):
                e = rel_err(gotg.cpu().double(), w64)
                self.report(tag + f' bwd_expanded det={det} g{k}', e <= tol, e)


def test_random_shapes(dev):
    sweep = _Sweep(dev)
    for i in range(CASES):
        sweep.forest_case(i)
        sweep.conv_case(i)
        sweep.expanded_case(i)
    assert not sweep.failures, sweep.failures
