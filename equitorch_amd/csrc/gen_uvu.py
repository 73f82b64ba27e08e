"""Emits ``generated/uvu_configs.inc``: straight-line device code for the channel-wise tensor product of
each registered irreps configuration.

For a configuration the Clebsch-Gordan table is a list of ``(coef, M, M1, M2, p)``.  Both bodies walk the
table path by path (the weight row of a path is fetched when the path starts and its gradient handed over
when the path ends).  The forward body evaluates, per weight path ``p`` and output row ``M``,

    t      = sum_{nnz in (p, M)} (coef * y[M2]) * x[M1]        (V channels per lane)
    out[M] += w[p] * t

and the backward body, per ``(p, M)`` segment,

    gw[p]  += g[M] * t                     gq = g[M] * w[p]
    gx[M1] += (coef * y[M2]) * gq          gy[M2] += coef * <x[M1], gq>_V

with every index a literal, so ``x``, ``w``, ``g`` and the accumulators live in registers.  Coefficients
are written as hexadecimal float literals of the fp32-rounded table values, the same bits the table tensors
of the Python API hold.

Run as ``python -m equitorch_amd.csrc.gen_uvu`` (done by the build step).
"""
from __future__ import annotations

import os
from collections import OrderedDict

import numpy as np

from .._tables import fingerprint, tp_coo
from ..irreps import Irreps
from ..utils import tp_infos

HERE = os.path.dirname(os.path.abspath(__file__))


def _sh(l):
    return Irreps.spherical_harmonics(l).short_repr()


# name -> (irreps_out, irreps_in1, irreps_in2, tp_infos kwargs)
CONFIGS = OrderedDict([
    ("sh1", (_sh(1), _sh(1), _sh(1), {})),
    ("sh2", (_sh(2), _sh(2), _sh(2), {})),
    ("sh3", (_sh(3), _sh(3), _sh(3), {})),
    ("so3_012_to_0123", ("0e+1e+2e+3e", "0e+1e+2e", "0e+1e+2e", {})),
])


def _lit(v: float) -> str:
    return float(np.float32(v)).hex() + "f"


def _opaque(m2s) -> str:
    """Per path, hide the harmonics it reads behind an empty asm statement.  Many (coefficient, harmonic)
    products recur in several paths; without this the optimiser computes each once and keeps it alive across
    the whole body, which costs far more registers than the multiplications it saves."""
    return "    " + " ".join(f'asm volatile("" : "+v"(yy[{m}]));' for m in m2s)


def sh_degree(irreps_in2) -> int:
    """L when the second operand has the layout of spherical harmonics of degrees 0..L (one irrep per degree, in
    order, any parity), else -1: only then can a kernel evaluate the operand from a vector."""
    ls = [ir.l for ir in Irreps(irreps_in2)]
    return len(ls) - 1 if ls == list(range(len(ls))) else -1


def table_arrays(coo) -> list:
    """The table itself as data members, so that the library can describe a compiled configuration to a caller
    that wants to match another table against it: fp32 coefficients and (M, M1, M2, p) per entry, table order."""
    T = coo.coef.shape[0]
    coefs = ", ".join(_lit(coo.coef[t]) for t in range(T))
    idx = ", ".join(f"{{{coo.M[t]}, {coo.M1[t]}, {coo.M2[t]}, {coo.p[t]}}}" for t in range(T))
    return [f"  static constexpr float COEF[{T}] = {{{coefs}}};",
            f"  static constexpr unsigned char IDX[{T}][4] = {{{idx}}};"]


def emit_config(name: str, coo, sh_lmax: int = -1) -> str:
    T = coo.coef.shape[0]
    # (p, M) segments, path-major: the weight row of a path is needed only while that path is evaluated, and
    # its gradient is complete when the path ends, so neither has to stay in registers.
    segs = OrderedDict()
    for t in range(T):
        segs.setdefault((int(coo.p[t]), int(coo.M[t])), []).append(t)
    by_path = OrderedDict()
    for (p, M), ts in sorted(segs.items()):
        by_path.setdefault(p, []).append((M, ts))
    L = []
    a = L.append
    a(f"struct TP_{name} {{")
    a(f"  static constexpr int D1 = {coo.D1}, D2 = {coo.D2}, DO = {coo.DO}, P = {coo.P}, NNZ = {T};")
    a(f"  static constexpr unsigned long long FINGERPRINT = 0x{fingerprint(coo):016x}ull;")
    a(f"  static constexpr unsigned long long FINGERPRINT_BF16 = 0x{fingerprint(coo, 'bf16'):016x}ull;")
    a(f"  static constexpr unsigned long long FINGERPRINT_F16 = 0x{fingerprint(coo, 'f16'):016x}ull;")
    a(f"  static constexpr const char* NAME = \"{name}\";")
    a(f"  static constexpr int SH_LMAX = {sh_lmax};  // second operand = harmonics of degrees 0..SH_LMAX (-1: not)")
    L.extend(table_arrays(coo))
    # ---- forward: o[M] += w[p] * sum_t (coef_t y[M2_t]) x[M1_t]
    a("  // wload(p, w): fetch the V channels of weight path p")
    a("  template <typename T, int V, class WLoad>")
    a("  __device__ __forceinline__ static void fwd(const T (&x)[D1][V], const T (&y)[D2], WLoad&& wload,")
    a("                                             T (&o)[DO][V]) {")
    a("    T t[V], w[V], yy[D2];")
    a("    for (int j = 0; j < D2; ++j) yy[j] = y[j];")
    for p, items in by_path.items():
        a(f"    wload({p}, w);")
        a(_opaque(sorted({int(coo.M2[t]) for _, ts in items for t in ts})))
        for M, ts in items:
            for n, t in enumerate(ts):
                op = "mulv" if n == 0 else "fmav"
                a(f"    {op}(t, T({_lit(coo.coef[t])}) * yy[{coo.M2[t]}], x[{coo.M1[t]}]);")
            a(f"    fmavv(o[{M}], w, t);")
    a("  }")
    # ---- backward
    a("  // gwsink(p, gw): consume the finished gradient of weight path p")
    a("  template <typename T, int V, class WLoad, class GwSink>")
    a("  __device__ __forceinline__ static void bwd(const T (&x)[D1][V], const T (&y)[D2], WLoad&& wload,")
    a("                                             const T (&g)[DO][V], T (&gx)[D1][V], T (&gy)[D2],")
    a("                                             GwSink&& gwsink) {")
    a("    T t[V], gq[V], w[V], gw[V], s, yy[D2];")
    a("    for (int j = 0; j < D2; ++j) yy[j] = y[j];")
    for p, items in by_path.items():
        a(f"    wload({p}, w);")
        a(_opaque(sorted({int(coo.M2[t]) for _, ts in items for t in ts})))
        for k, (M, ts) in enumerate(items):
            a(f"    mulvv(gq, g[{M}], w);")
            for n, t in enumerate(ts):
                c, m1, m2 = _lit(coo.coef[t]), coo.M1[t], coo.M2[t]
                a(f"    s = T({c}) * yy[{m2}];")
                a(f"    {'mulv' if n == 0 else 'fmav'}(t, s, x[{m1}]);")
                a(f"    fmav(gx[{m1}], s, gq);")
                a(f"    gy[{m2}] = fma(T({c}), dotv(x[{m1}], gq), gy[{m2}]);")
            a(f"    {'mulvv' if k == 0 else 'fmavv'}(gw, g[{M}], t);")
        a(f"    gwsink({p}, gw);")
    a("  }")
    a("};")
    return "\n".join(L)


def main(out_dir: str = None) -> str:
    out_dir = out_dir or os.path.join(HERE, "generated")
    os.makedirs(out_dir, exist_ok=True)
    chunks = ["// Generated by equitorch_amd/csrc/gen_uvu.py; do not edit.", ""]
    for name, (io, i1, i2, kw) in CONFIGS.items():
        coo = tp_coo(tp_infos(Irreps(io), Irreps(i1), Irreps(i2), **kw)[0])
        chunks.append(f"// {name}: {i1} x {i2} -> {io} {kw if kw else ''}")
        chunks.append(emit_config(name, coo, sh_degree(i2)))
        chunks.append("")
    chunks.append("#define CGTP_FOREACH_UVU_CONFIG(X) \\")
    chunks.append(" \\\n".join(f"  X(TP_{n})" for n in CONFIGS))
    chunks.append("")
    path = os.path.join(out_dir, "uvu_configs.inc")
    text = "\n".join(chunks)
    if not os.path.exists(path) or open(path).read() != text:
        with open(path, "w") as f:
            f.write(text)
    return path


if __name__ == "__main__":
    print(main())
