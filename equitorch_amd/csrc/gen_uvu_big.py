"""Emits ``generated/uvu_big_configs.inc``: the channel-wise tensor product, one channel per lane, for row-mode
launches of every registered configuration and for configurations whose table is too large for the
register-resident bodies of ``gen_uvu`` (hundreds of weight rows, thousands of coefficients).

One lane owns one channel.  The forward walks the table output irrep by output irrep (only the 2l+1 accumulator
rows of that irrep are live), the backward input irrep by input irrep (only that irrep's rows of x and grad_x are
live, next to all of y, grad_y and grad_out: at lmax = 6 that is 173 registers instead of 209 for the walk by
output irrep, and the body needs no scratch memory), inside an irrep path by path.  A path's weight is a single
register, taken from a ring of ``RING`` registers that is refilled ``RING`` paths ahead so that the per-row weight
stream never waits for memory.  Per path the forward evaluates

    t = y[b] * x[a]   once per (a, b) pair,      i[M] += coef * t,      o[M] += w[p] * i[M]

and the backward contracts the coefficients with the rows of ``grad_out`` first, once per (a, b) pair,

    v = sum_M coef * g[M]        s[a] += y[b] * v        gy[b] += (w[p] * x[a]) * v
    gw[p] = sum_a x[a] * s[a]    gx[a] += w[p] * s[a]

so that a coefficient costs one instruction and a pair two (the forward intermediate is not rebuilt).  Every
index is a literal and every coefficient the hexadecimal literal of the fp32 table value.
"""
from __future__ import annotations

import os
from collections import OrderedDict

from .._tables import fingerprint, tp_coo
from ..irreps import Irreps, irrep_segments
from ..utils import tp_infos
from .gen_uvu import _lit, _sh, table_arrays

HERE = os.path.dirname(os.path.abspath(__file__))
RING = 8

CONFIGS = OrderedDict([
    ("sh1", (_sh(1), _sh(1), _sh(1), {})),
    ("sh2", (_sh(2), _sh(2), _sh(2), {})),
    ("sh3", (_sh(3), _sh(3), _sh(3), {})),
    ("sh4", (_sh(4), _sh(4), _sh(4), {})),
    ("sh5", (_sh(5), _sh(5), _sh(5), {})),
    ("sh6", (_sh(6), _sh(6), _sh(6), {})),
    ("so3_012_to_0123", ("0e+1e+2e+3e", "0e+1e+2e", "0e+1e+2e", {})),
    ("so3_2", ("0e+1e+2e", "0e+1e+2e", "0e+1e+2e", {})),
    ("so3_3", ("0e+1e+2e+3e", "0e+1e+2e+3e", "0e+1e+2e+3e", {})),
    ("so3_4", ("0e+1e+2e+3e+4e", "0e+1e+2e+3e+4e", "0e+1e+2e+3e+4e", {})),
])


def extra_configs() -> OrderedDict:
    """Configurations a user registers in ``extra_uvu_configs.json`` next to this file:
    ``{"name": ["irreps_out", "irreps_in1", "irreps_in2"], ...}`` (names: C identifiers).  They are compiled into the
    library by the next build like the ones above."""
    import json
    path = os.path.join(HERE, "extra_uvu_configs.json")
    out = OrderedDict()
    if os.path.exists(path):
        with open(path) as f:
            for name, (io, i1, i2) in json.load(f).items():
                if not name.isidentifier():
                    raise ValueError(f"{path}: configuration name {name!r} is not an identifier")
                out[name] = (io, i1, i2, {})
    return out


def _pin(names) -> str:
    """An empty asm that takes the accumulators as in/out operands, in chunks of 12: without it the optimiser
    sinks updates towards the final store and keeps whole paths of temporaries alive."""
    names = list(names)
    out = []
    for i in range(0, len(names), 12):
        out.append('asm volatile("" : ' + ", ".join(f'"+v"({n})' for n in names[i:i + 12]) + ");")
    return " ".join(out)


def _grouped(terms, key):
    d = OrderedDict()
    for t in sorted(terms, key=key):
        d.setdefault(key(t), []).append(t)
    return d


def emit_config(name: str, coo, seg_out, seg_in1) -> str:
    T = coo.coef.shape[0]
    term = [(int(coo.p[t]), int(coo.M[t]), int(coo.M1[t]), int(coo.M2[t]), _lit(coo.coef[t])) for t in range(T)]
    # execution order: output irrep blocks, inside a block the paths in table order
    blocks = []
    for b0, b1 in zip(seg_out[:-1], seg_out[1:]):
        paths = sorted({p for p, M, _, _, _ in term if b0 <= M < b1})
        if paths:
            blocks.append((list(range(b0, b1)), paths))
    order = [p for _, paths in blocks for p in paths]
    assert sorted(order) == list(range(coo.P))
    pos = {p: k for k, p in enumerate(order)}
    by_path = {p: [t for t in term if t[0] == p] for p in order}

    L = []
    a = L.append
    a(f"struct TPB_{name} {{")
    a(f"  static constexpr int D1 = {coo.D1}, D2 = {coo.D2}, DO = {coo.DO}, P = {coo.P}, NNZ = {T};")
    a(f"  static constexpr unsigned long long FINGERPRINT = 0x{fingerprint(coo):016x}ull;")
    a(f"  static constexpr unsigned long long FINGERPRINT_BF16 = 0x{fingerprint(coo, 'bf16'):016x}ull;")
    a(f"  static constexpr unsigned long long FINGERPRINT_F16 = 0x{fingerprint(coo, 'f16'):016x}ull;")
    a(f"  static constexpr const char* NAME = \"{name}\";")
    L.extend(table_arrays(coo))

    def ring_prologue():
        for k in range(min(RING, len(order))):
            a(f"    float wq{k} = wload({order[k]});")

    def ring_take(p):
        k = pos[p]
        a(f"      const float w = wq{k % RING};")
        if k + RING < len(order):
            a(f"      wq{k % RING} = wload({order[k + RING]});")

    def opaque(ys):
        a("      " + " ".join(f'asm volatile("" : "+v"(yy[{m}]));' for m in sorted(ys)))

    # ---- forward ---------------------------------------------------------------------------------------------
    a("  // wload(p): this lane's channel of weight path p; store(M, v): one finished output row")
    a("  template <class WLoad, class Store>")
    a("  __device__ __forceinline__ static void fwd(const float (&x)[D1], const float (&y)[D2], WLoad&& wload,")
    a("                                             Store&& store) {")
    a("    float yy[D2];")
    a("    for (int j = 0; j < D2; ++j) yy[j] = y[j];")
    ring_prologue()
    for rows, paths in blocks:
        a("    {")
        a("      float " + ", ".join(f"o{M} = 0.f" for M in rows) + ";")
        for p in paths:
            ms = sorted({M for _, M, _, _, _ in by_path[p]})
            a("      {")
            ring_take(p)
            opaque({b for _, _, _, b, _ in by_path[p]})
            a("      float " + ", ".join(f"i{M}" for M in ms) + ";")
            seen = set()
            for (aa, b), ts in _grouped(by_path[p], lambda t: (t[2], t[3])).items():
                ops = []
                for _, M, _, _, c in ts:
                    ops.append(f"i{M} {'+=' if M in seen else '='} {c} * t;")
                    seen.add(M)
                a(f"      {{ const float t = yy[{b}] * x[{aa}]; " + " ".join(ops) + " }")
            a("      " + " ".join(f"o{M} += w * i{M};" for M in ms))
            a("      " + _pin(f"o{M}" for M in ms))
            a("      }")
        for M in rows:
            a(f"      store({M}, o{M});")
        a("    }")
    a("  }")

    # ---- backward --------------------------------------------------------------------------------------------
    # Walks the table input irrep by input irrep: of x and grad_x only the 2l+1 rows of the current irrep are
    # live (and the next irrep's rows of x, requested one block ahead); y, grad_y and grad_out stay whole.
    blocks_in = []
    for b0, b1 in zip(seg_in1[:-1], seg_in1[1:]):
        paths = sorted({p for p, _, aa, _, _ in term if b0 <= aa < b1})
        if paths:
            blocks_in.append((list(range(b0, b1)), paths))
    order = [p for _, paths in blocks_in for p in paths]
    assert sorted(order) == list(range(coo.P))
    pos = {p: k for k, p in enumerate(order)}
    a("  // xload(a): this lane's channel of row a of x; wload(p): of weight path p; g: the rows of grad_out;")
    a("  // gxstore(a, v): a finished row of grad_x; gwsink(p, v): gradient of weight path p; gy: accumulated in place")
    a("  // (this lane's channel only, the caller sums over channels)")
    a("  template <class XLoad, class WLoad, class GxStore, class GwSink>")
    a("  __device__ __forceinline__ static void bwd(XLoad&& xload, const float (&y)[D2], WLoad&& wload,")
    a("                                             const float (&g)[DO], GxStore&& gxstore, float (&gy)[D2],")
    a("                                             GwSink&& gwsink) {")
    a("    float yy[D2], gg[DO];")
    a("    for (int j = 0; j < D2; ++j) yy[j] = y[j];")
    a("    for (int j = 0; j < DO; ++j) gg[j] = g[j];")
    ring_prologue()
    for aa in blocks_in[0][0]:
        a(f"    float x{aa} = xload({aa});")
    for bi, (rows, paths) in enumerate(blocks_in):
        if bi + 1 < len(blocks_in):
            for aa in blocks_in[bi + 1][0]:
                a(f"    float x{aa} = xload({aa});")
        a("    {")
        a("      float " + ", ".join(f"gx{aa} = 0.f" for aa in rows) + ";")
        for p in paths:
            ts_p = by_path[p]
            a("      {")
            ring_take(p)
            opaque({b for _, _, _, b, _ in ts_p})
            a("      " + " ".join(f'asm volatile("" : "+v"(gg[{m}]));' for m in sorted({t[1] for t in ts_p})))
            a("      float gwp;")
            for ai, (aa, ts_a) in enumerate(_grouped(ts_p, lambda t: t[2]).items()):
                a(f"      {{ const float xw = w * x{aa}; float s;")
                for bi_, (b, ts) in enumerate(_grouped(ts_a, lambda t: t[3]).items()):
                    v = " + ".join(f"{c} * gg[{M}]" for _, M, _, _, c in ts)
                    pins = f' asm volatile("" : "+v"(s), "+v"(gy[{b}]));'
                    a(f"        {{ const float v = {v}; s {'+=' if bi_ else '='} yy[{b}] * v; gy[{b}] += xw * v;{pins} }}")
                a(f"        gwp {'+=' if ai else '='} x{aa} * s; gx{aa} += w * s; }}")
            a(f"      gwsink({p}, gwp);")
            a("      " + _pin(f"gx{m}" for m in sorted({t[2] for t in ts_p})))
            a("      }")
        for aa in rows:
            a(f"      gxstore({aa}, gx{aa});")
        a("    }")
    a("  }")
    a("};")
    return "\n".join(L)


def main(out_dir: str = None) -> str:
    out_dir = out_dir or os.path.join(HERE, "generated")
    os.makedirs(out_dir, exist_ok=True)
    chunks = ["// Generated by equitorch_amd/csrc/gen_uvu_big.py; do not edit.", ""]
    configs = OrderedDict(CONFIGS)
    configs.update(extra_configs())
    seen = {}
    for name, (io, i1, i2, kw) in configs.items():
        coo = tp_coo(tp_infos(Irreps(io), Irreps(i1), Irreps(i2), **kw)[0])
        fp = fingerprint(coo)
        if fp in seen:
            raise ValueError(f"configuration {name} has the same table as {seen[fp]}")
        seen[fp] = name
        chunks.append(f"// {name}: {i1} x {i2} -> {io}")
        chunks.append(emit_config(name, coo, irrep_segments(Irreps(io)), irrep_segments(Irreps(i1))))
        chunks.append("")
    chunks.append("#define CGTP_FOREACH_UVU_BIG_CONFIG(X) \\")
    chunks.append(" \\\n".join(f"  X(TPB_{n})" for n in configs))
    chunks.append("")
    path = os.path.join(out_dir, "uvu_big_configs.inc")
    text = "\n".join(chunks)
    if not os.path.exists(path) or open(path).read() != text:
        with open(path, "w") as f:
            f.write(text)
    return path


if __name__ == "__main__":
    print(main())
