"""Writes the golden table fixtures ``tp_tables.npz`` and ``scale_tables.npz`` in this directory.

Run once, in the build container only (it needs ``/root/reference``); the fixtures it writes are committed
and are the only thing that travels.  It loads the reference's own table-building chain
(``equitorch/constants``, ``irreps``, ``structs``, ``utils/_indices.py``, ``utils/_structs.py``) without
executing ``equitorch/__init__.py`` (which would pull in modules that need packages absent here), calls
``tp_infos`` / ``sparse_scale_infos`` and stores every tensor field as a numpy array.

What the fixtures pin that mathematics alone does not: the fp32 bits of every ``scale`` entry
(``float(sympy) * norm`` rounded by ``torch.tensor``), the exact sparsity pattern kept by ``!= 0.0``, and
the identity-collapse (``None``) decisions of every index/segment field.

Key layout: ``<case>/<direction>/<info field>/<tensor field>``; a field that is ``None`` in the reference is
recorded in ``<case>/<direction>/<info field>/__none__`` (array of field names); ``out_size`` is stored too.
"""
import importlib
import json
import os
import sys
import types
import typing

import numpy as np
import torch

REF = "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))

TP_CASES = {
    # name: (irreps_out, irreps1, irreps2, kwargs)
    "sh2": ("0e+1o+2e", "0e+1o+2e", "0e+1o+2e", {}),
    "sh3": ("0e+1o+2e+3o", "0e+1o+2e+3o", "0e+1o+2e+3o", {}),
    "sh6": ("0e+1o+2e+3o+4e+5o+6e",) * 3 + ({},),
    "gradcheck": ("0e+1e+2e+3e", "0e+1e+2e", "0e+1e+2e", {}),
    "so3_13": ((1, 3), (1, 3), (1, 3), {}),
    "sh2_nonorm": ("0e+1o+2e", "0e+1o+2e", "0e+1o+2e", {"path_norm": False}),
    "sh2_chnorm": ("0e+1o+2e", "0e+1o+2e", "0e+1o+2e", {"channel_norm": True, "channel_scale": 128 ** -0.5}),
    "mult": ("2x0e+1o+2x2e", "0e+2x1o", "0e+1o+2e", {}),
    "sh1_to_2": ("0e+1o+2e", "0e+1o", "0e+1o", {}),
    "explicit_path": ("0e+1o+2e", "0e+1o+2e", "0e+1o+2e", {"path": [(0, 1, 1), (1, 1, 2), (2, 0, 2), (2, 2, 2)]}),
}


def load_reference():
    if not hasattr(typing, "override"):  # Python < 3.12: a no-op marker decorator
        typing.override = lambda f: f
    pkg = types.ModuleType("equitorch")
    pkg.__path__ = [os.path.join(REF, "equitorch")]
    sys.modules["equitorch"] = pkg
    utils = types.ModuleType("equitorch.utils")
    utils.__path__ = [os.path.join(REF, "equitorch", "utils")]
    sys.modules["equitorch.utils"] = utils
    for name in ("equitorch.irreps", "equitorch.constants", "equitorch.structs", "equitorch.utils._indices"):
        importlib.import_module(name)
    return importlib.import_module("equitorch.utils._structs")


def dump_info(prefix, info, out):
    none_fields = []
    for field in info._fields:
        v = getattr(info, field)
        if isinstance(v, torch.Tensor):
            out[f"{prefix}/{field}"] = v.numpy()
            out[f"{prefix}/{field}/dtype"] = np.array(str(v.dtype))
        elif v is None:
            none_fields.append(field)
        elif isinstance(v, int):
            out[f"{prefix}/{field}"] = np.array(v, dtype=np.int64)
        else:
            raise TypeError((prefix, field, type(v)))
    out[f"{prefix}/__none__"] = np.array(none_fields, dtype="U32")


def main():
    ref = load_reference()
    from equitorch.irreps import Irreps

    out = {}
    meta = {}
    for name, (io, i1, i2, kw) in TP_CASES.items():
        fwd, b1, b2, num_paths = ref.tp_infos(Irreps(io), Irreps(i1), Irreps(i2), **kw)
        for dname, tp in (("fwd", fwd), ("bwd1", b1), ("bwd2", b2)):
            for field in tp._fields:
                v = getattr(tp, field)
                if field == "out_size":
                    out[f"{name}/{dname}/out_size"] = np.array(v, dtype=np.int64)
                else:
                    dump_info(f"{name}/{dname}/{field}", v, out)
        meta[name] = {"irreps_out": str(io), "irreps1": str(i1), "irreps2": str(i2), "kwargs": kw,
                      "num_paths": num_paths}
        print(name, "paths", num_paths, "nnz", fwd.info_Mij_fwd.scale.numel())
    np.savez_compressed(os.path.join(HERE, "tp_tables.npz"), **out)
    with open(os.path.join(HERE, "tp_tables_meta.json"), "w") as f:
        json.dump(meta, f, indent=1)

    # sparse_scale_infos on small graphs: the dst-sorted edge permutation / CSR pointer used for the
    # edge -> node scatter-sum and its transpose.
    out = {}
    g = torch.Generator().manual_seed(0)
    for name, (n_nodes, n_edges, scaled) in {"g8_40": (8, 40, False), "g5_12_scaled": (5, 12, True),
                                             "g64_700": (64, 700, False), "g6_4_sparse": (6, 4, False)}.items():
        dst = torch.randint(0, n_nodes, (n_edges,), generator=g).tolist()
        scale = torch.randn(n_edges, generator=g).tolist() if scaled else None
        fwd, bwd = ref.sparse_scale_infos(index=list(range(n_edges)), index_out=dst, scale=scale,
                                          out_size=n_nodes, in_size=n_edges)
        out[f"{name}/dst"] = np.array(dst, dtype=np.int64)
        if scaled:
            out[f"{name}/scale_in"] = np.array(scale, dtype=np.float64)
        out[f"{name}/n_nodes"] = np.array(n_nodes)
        dump_info(f"{name}/fwd", fwd, out)
        dump_info(f"{name}/bwd", bwd, out)
    np.savez_compressed(os.path.join(HERE, "scale_tables.npz"), **out)


if __name__ == "__main__":
    main()
