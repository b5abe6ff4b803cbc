"""Writes tests/golden/*.npz from the reference's own CPU build (oracle/_ref/hingetree_cpp.so, made by
`make -C oracle ref` from the sources under /root/reference). Run in the authoring container only:

    python tests/golden/make_golden.py            # everything
    python tests/golden/make_golden.py tiles      # only the contract / expand fixtures
    python tests/golden/make_golden.py mix        # only the forest -> linear fixtures
    python tests/golden/make_golden.py snapshot   # only the trained-snapshot fixture

Each file holds seeded inputs and the reference's outputs for one small case; tests compare the oracle (CPU) and the
HIP path (GPU) against them. The fixtures are data only.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

from conftest import make_conv, make_forest  # noqa: E402
from oracle import hinge_oracle as ho  # noqa: E402

FOREST_CASES = {
    # name: (B, F, Kd, T, D, Md, fern, dtype, x_dist)
    "tree_f32_plain": (12, 16, [], 6, 4, [], False, torch.float32, "normal"),
    "tree_f32_m10": (9, 20, [], 5, 5, [10], False, torch.float32, "uniform"),
    "tree_f32_inner": (4, 6, [3, 2], 3, 3, [2, 2], False, torch.float32, "normal"),
    "tree_f64_m3": (8, 10, [], 4, 6, [3], False, torch.float64, "normal"),
    "fern_f32_m1": (12, 16, [], 6, 5, [1], True, torch.float32, "normal"),
    "fern_f64_inner": (3, 7, [5], 4, 4, [2], True, torch.float64, "normal"),
}

CONV_CASES = {
    # name: (B, C, Cout, size, D, Md, kernel, stride, padding, dilation, fern, dtype)
    "conv1d_tree": (2, 3, 4, [11], 3, [], [3], [2], [1], [1], False, torch.float32),
    "conv2d_tree": (2, 3, 4, [7, 6], 3, [], [3, 3], [1, 1], [1, 1], [1, 1], False, torch.float32),
    "conv2d_tree_m3_dil": (1, 2, 3, [9, 8], 2, [3], [3, 2], [2, 1], [2, 0], [2, 2], False, torch.float64),
    "conv3d_fern": (1, 2, 2, [5, 4, 6], 3, [2], [2, 2, 3], [1, 2, 1], [0, 1, 1], [1, 1, 1], True, torch.float32),
}

TILE_CASES = {
    # name: (shape, window, padding, dtype)
    "tiles2d_f32": ([2, 3, 9, 11], [4, 3], [1, 2], torch.float32),
    "tiles2d_u8_exact": ([1, 2, 8, 12], [2, 4], [0, 0], torch.uint8),
    "tiles3d_i16": ([2, 1, 5, 6, 7], [2, 3, 2], [1, 0, 1], torch.int16),
    "tiles3d_f64_big_pad": ([1, 2, 4, 5, 3], [3, 2, 2], [2, 1, 2], torch.float64),
}

MIX_CASES = {
    # name: (B, F, Kd, T, D, Md, O, fern, dtype)
    "mix_tree_f32": (10, 12, [], 7, 4, [], 5, False, torch.float32),
    "mix_tree_f32_inner": (3, 6, [2, 3], 4, 3, [3], 6, False, torch.float32),
    "mix_fern_f32_m2": (8, 9, [], 5, 4, [2], 3, True, torch.float32),
    "mix_fern_f64_inner": (4, 7, [4], 3, 3, [], 2, True, torch.float64),
}


def write_mix(ref):
    for name, (B, F, Kd, T, D, Md, O, fern, dtype) in MIX_CASES.items():
        x, thr, ordn, w, _ = make_forest(B, F, Kd, T, D, Md, fern, dtype, seed=31)
        g = torch.Generator().manual_seed(32)
        lin = torch.randn([O, T], generator=g, dtype=dtype) / T ** 0.5
        bias = torch.randn([O], generator=g, dtype=dtype)
        pre = "fern_" if fern else "tree_"
        out = getattr(ref, pre + "fused_linear_forward")(x, thr, ordn, w, lin, bias)
        gout = torch.randn(out.shape, generator=g, dtype=dtype)
        dx, dthr, _, dw, dlin, dbias = getattr(ref, pre + "fused_linear_backward")(
            x, True, thr, True, ordn, False, w, True, lin, True, bias, True, gout)
        np.savez_compressed(os.path.join(HERE, name + ".npz"), fern=np.int64(fern), x=x.numpy(), thr=thr.numpy(),
                            ord=ordn.numpy(), w=w.numpy(), lin=lin.numpy(), bias=bias.numpy(), gout=gout.numpy(),
                            out=out.numpy(), dx=dx.numpy(), dthr=dthr.numpy(), dw=dw.numpy(), dlin=dlin.numpy(),
                            dbias=dbias.numpy())

SNAPSHOT = ("/root/reference/rcc/Models/snapshots_unweighted_easyhard_deterministic_hingeforest_depth7_vggblock3_"
            "randomSplit1/epoch_549.pt")
SNAPSHOT_TREES = 3


def write_snapshot(ref):
    """Parameters of the first trees of the forest in one of the trained segmentation snapshots the reference ships
    (data: thresholds, ordinals stored as float32 as old versions of the reference did, leaf weights [.., 8, 8]), and
    what the reference's CPU build computes from them for a seeded input: forest output, leaf map, and the image the
    8 x 8 leaf patches expand to. Read with the loader that executes nothing from the file."""
    sd = torch.load(SNAPSHOT, map_location="cpu", weights_only=True)
    thr = sd["forest.thresholds"][:SNAPSHOT_TREES].contiguous()
    ordf = sd["forest.ordinals"][:SNAPSHOT_TREES].contiguous()
    w = sd["forest.weights"][:SNAPSHOT_TREES].contiguous()
    assert ordf.dtype == torch.float32 and torch.equal(ordf, ordf.round())
    x = torch.randn([2, 100, 3, 4], generator=torch.Generator().manual_seed(41))
    ordn = ordf.long()
    out = ref.tree_forward(x, thr, ordn, w)
    leaf = ref.tree_leafmap(x, thr, ordn, w)
    image = ref.expand(out, [0, 0])
    np.savez_compressed(os.path.join(HERE, "snapshot_forest_subset.npz"), thr=thr.numpy(), ord_float=ordf.numpy(),
                        w=w.numpy(), x=x.numpy(), out=out.numpy(), leaf=leaf.numpy(), image=image.numpy())


def write_tiles(ref):
    for name, (shape, window, padding, dtype) in TILE_CASES.items():
        g = torch.Generator().manual_seed(23)
        x = (200.0 * torch.rand(shape, generator=g) - 50.0).to(dtype)
        tiles = ref.contract(x, window, padding)
        image = ref.expand(tiles, padding)
        np.savez_compressed(os.path.join(HERE, name + ".npz"), x=x.numpy(), window=np.array(window),
                            padding=np.array(padding), tiles=tiles.numpy(), image=image.numpy())


def main():
    ref = ho.reference_module()
    if ref is None:
        raise SystemExit("oracle/_ref/hingetree_cpp.so is missing: run `make -C oracle ref` first")
    only = sys.argv[1] if len(sys.argv) == 2 else None
    if only in (None, "tiles"):
        write_tiles(ref)
    if only in (None, "mix"):
        write_mix(ref)
    if only in (None, "snapshot"):
        write_snapshot(ref)
    if only is not None:
        print("wrote", sorted(f for f in os.listdir(HERE) if f.startswith(only)))
        return
    for name, (B, F, Kd, T, D, Md, fern, dtype, dist) in FOREST_CASES.items():
        x, thr, ordn, w, gout = make_forest(B, F, Kd, T, D, Md, fern, dtype, seed=11, x_dist=dist)
        pre = "fern_" if fern else "tree_"
        if not fern:
            getattr(ref, pre + "fix_thresholds")(thr, ordn, w)
        out = getattr(ref, pre + "forward")(x, thr, ordn, w)
        dx, dthr, _, dw = getattr(ref, pre + "backward")(x, True, thr, True, ordn, False, w, True, gout)
        leaf = getattr(ref, pre + "leafmap")(x, thr, ordn, w)
        margin, sel = getattr(ref, pre + "marginmap")(x, thr, ordn, w)
        reach = getattr(ref, pre + "reachability")(x, thr, ordn, w)
        np.savez_compressed(os.path.join(HERE, name + ".npz"), fern=np.int64(fern), x=x.numpy(), thr=thr.numpy(),
                            ord=ordn.numpy(), w=w.numpy(), gout=gout.numpy(), out=out.numpy(), dx=dx.numpy(),
                            dthr=dthr.numpy(), dw=dw.numpy(), leaf=leaf.numpy(), margin=margin.numpy(), sel=sel.numpy(),
                            reach=reach.numpy())
    for name, (B, C, Cout, size, D, Md, ker, st, pad, dil, fern, dtype) in CONV_CASES.items():
        x, thr, ordn, w = make_conv(B, C, Cout, size, D, Md, ker, fern, dtype, seed=5)
        nd = len(size)
        pre = ("fern_" if fern else "tree_") + f"conv{nd}d_"
        out = getattr(ref, pre + "forward")(x, thr, ordn, w, ker, st, pad, dil)
        gout = torch.randn(out.shape, generator=torch.Generator().manual_seed(77), dtype=dtype)
        dx, dthr, _, dw = getattr(ref, pre + "backward")(x, True, thr, True, ordn, False, w, True, gout, ker, st, pad, dil)
        np.savez_compressed(os.path.join(HERE, name + ".npz"), fern=np.int64(fern), x=x.numpy(), thr=thr.numpy(),
                            ord=ordn.numpy(), w=w.numpy(), gout=gout.numpy(), out=out.numpy(), dx=dx.numpy(),
                            dthr=dthr.numpy(), dw=dw.numpy(), kernel=np.array(ker), stride=np.array(st),
                            padding=np.array(pad), dilation=np.array(dil))
    # threshold repair: inputs that need fixing, and the reference's in-place result
    g = torch.Generator().manual_seed(3)
    thr = 6.0 * torch.rand([12, 31], generator=g) - 3.0
    ordn = torch.randint(0, 3, [12, 31], generator=g)
    w = torch.randn([12, 32], generator=g)
    before = thr.clone()
    ok_before = ref.tree_check_thresholds(thr, ordn, w)
    changed = ref.tree_fix_thresholds(thr, ordn, w)
    ok_after = ref.tree_check_thresholds(thr, ordn, w)
    np.savez_compressed(os.path.join(HERE, "fix_thresholds.npz"), before=before.numpy(), ord=ordn.numpy(), w=w.numpy(),
                        after=thr.numpy(), ok_before=np.array(ok_before), changed=np.array(changed),
                        ok_after=np.array(ok_after))
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))


if __name__ == "__main__":
    main()
