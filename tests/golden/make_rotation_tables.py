"""Writes the golden fixture ``rotation_tables.npz``: the reference's own ``wigner_d_info`` and ``so2_linear_infos``
tables for a few irreps.

Run once, in the build container only (it needs ``/root/reference``), like ``make_tables.py`` whose loader it uses;
only the tensors it stores travel.  What these fixtures pin that no closed form does: the fp32 bits of the J-matrix
entries (``float()`` of symbolic values, entries below 1e-9 dropped) and the path-count normalisation of the SO(2)
linear tables, which follows the bookkeeping of the reference's builder rather than a formula.
"""
import os

import numpy as np

from make_tables import HERE, dump_info, load_reference

WIGNER_CASES = {"sh2": "0e+1o+2e", "so3_04": (0, 4), "odd13": "1o+3o", "mult": "2x1o+2e"}
SO2_CASES = {
    "sh2": ("0e+1o+2e", "0e+1o+2e", {}),
    "sh3_to_2": ("0e+1o+2e", "0e+1o+2e+3o", {}),
    "mult": ("1o+2e", "2x1o+2e+0e", {}),
    "nonorm": ("0e+1o+2e", "0e+1o+2e", {"path_norm": False}),
    "chnorm": ("0e+1o+2e", "0e+1o+2e", {"channel_norm": True, "channel_scale": 0.125}),
    "path": ("0e+1o+2e", "0e+1o+2e", {"path": [(0, 0), (1, 1), (2, 1), (2, 2)]}),
}


def main():
    ref = load_reference()
    from equitorch.irreps import Irreps
    out = {}
    for name, irr in WIGNER_CASES.items():
        info = ref.wigner_d_info(Irreps(irr))
        for field in ("j_matrix_info", "rotate_z_info_fwd", "rotate_z_info_bwd_input", "rotate_z_info_bwd_cs"):
            dump_info(f"wigner/{name}/{field}", getattr(info, field), out)
        out[f"wigner/{name}/sign"] = info.sign.numpy()
        out[f"wigner/{name}/max_m"] = np.array(info.max_m, dtype=np.int64)
        print("wigner", name, info.j_matrix_info.scale.numel(), info.rotate_z_info_fwd.scale.numel())
    for name, (io, ii, kw) in SO2_CASES.items():
        fwd, b1, b2, n = ref.so2_linear_infos(Irreps(io), Irreps(ii), **kw)
        for dname, info in (("fwd", fwd), ("bwd1", b1), ("bwd2", b2)):
            dump_info(f"so2/{name}/{dname}", info, out)
        out[f"so2/{name}/num_weights"] = np.array(n, dtype=np.int64)
        print("so2", name, n, fwd.scale.numel())
    np.savez_compressed(os.path.join(HERE, "rotation_tables.npz"), **out)


if __name__ == "__main__":
    main()
