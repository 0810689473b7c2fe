"""Cuts the data-only fixture tests/golden/garden_subset.npz out of the reference's
assets/test_garden.npz (means, colours and three real cameras of the "garden" scene).

    python tests/golden/make_garden_subset.py [/root/reference/assets/test_garden.npz]

Runs in the build container only (the reference checkout does not travel to the GPU box); the
.npz it writes is committed.  The file is opened with numpy's default allow_pickle=False.  Kept:
the crop to [-2, 2]^3 that the reference's loader applies before every test
(gsplat/_helper.py:31-36), thinned to every third point so that the fixture stays below
1 MB; the cameras, intrinsics and image size unchanged.  Nothing else of the reference is read.
"""
import os
import sys

import numpy as np

SRC = sys.argv[1] if len(sys.argv) > 1 else "/root/reference/assets/test_garden.npz"
DST = os.path.join(os.path.dirname(os.path.abspath(__file__)), "garden_subset.npz")
STRIDE = 3

data = np.load(SRC)  # allow_pickle=False
means = data["means3d"].astype(np.float32)
colors = data["colors"].astype(np.uint8)
sel = ((means >= -2.0) & (means <= 2.0)).all(-1)
means, colors = means[sel][::STRIDE], colors[sel][::STRIDE]
np.savez_compressed(DST, means3d=means, colors=colors, viewmats=data["viewmats"].astype(np.float32),
                    Ks=data["Ks"].astype(np.float32), height=np.int64(data["height"]),
                    width=np.int64(data["width"]), stride=np.int64(STRIDE), cropped=np.int64(sel.sum()))
print(DST, means.shape, colors.shape, os.path.getsize(DST), "bytes")
