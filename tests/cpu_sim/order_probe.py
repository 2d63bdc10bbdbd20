"""usage: python tests/cpu_sim/order_probe.py out.npz — one small scene through both footprints (forward and backward,
16x16 and 8x8 tiles) in the simulator, all outputs saved. tests/test_sim_kernels.py runs it under different
INPC_SIM_ORDER settings and compares the files bit for bit."""
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent.parent
sys.path.insert(0, str(ROOT))

from inpc_amd import _lib, synthetic  # noqa: E402
from tests import helpers as H  # noqa: E402
from tests.cpu_sim import simulated_device  # noqa: E402


def main(path):
    out = {}
    with simulated_device():
        for name, tile, channels in (("bilinear16", 16, 8), ("bilinear8", 8, 4)):
            n = 30000
            hv = synthetic.rotated_camera(203, 131, 180.0, 2.4, 0.2, -0.1)
            pos = synthetic.cube_points(n, 1.6, 5)
            pos[:4000] = pos[4000:8000]   # duplicates: equal depth keys, ties in the tile sort
            feats, opac = synthetic.point_attributes(n, channels, "normal", 6)
            rng = np.random.default_rng(1)
            run = H.RasterRun(hv, pos, feats, opac, tile, channels, _lib.FEAT_DIRECT_F32).forward()
            o = run.outputs()
            gi = rng.normal(0, 1e-2, o["image"].shape).astype(np.float32)
            ga = rng.normal(0, 1e-2, o["alpha"].shape).astype(np.float32)
            gf, go = run.backward(gi, ga)
            out.update({f"{name}_image": o["image"], f"{name}_alpha": o["alpha"],
                        f"{name}_blending_weights": o["blending_weights"], f"{name}_grad_features": gf,
                        f"{name}_grad_opacities": go})
            grun = H.GaussianRun(hv, pos, feats, opac, tile, channels, _lib.FEAT_DIRECT_F32, max_instances=40 * n).forward()
            o = grun.outputs()
            gf, go = grun.backward(gi, ga)
            name = name.replace("bilinear", "gaussian")
            out.update({f"{name}_image": o["image"], f"{name}_alpha": o["alpha"],
                        f"{name}_blending_weights": o["blending_weights"], f"{name}_grad_features": gf,
                        f"{name}_grad_opacities": go})
    np.savez(path, **out)


if __name__ == "__main__":
    main(sys.argv[1])
