"""Emits ``generated/uv_configs.inc``: the per-configuration bodies of the fully connected ("uv") tensor product
on the matrix cores.

Evaluation order is weight-first: for every weight path ``p`` and every row ``a`` of the channelled input that the
path reads, two accumulator tiles ``Z[w, n] = sum_u Wt[p][w, u] * x[n, a, u]`` (2 x 16 output channels x 16 samples,
K = C_in, bf16 MFMA with fp32 accumulation), then the Clebsch-Gordan stage as fp32 FMAs on accumulator tiles,
``out[m] += (coef * y[n, b]) * Z`` — in the MFMA accumulator layout every lane belongs to one sample, so the
harmonic ``y[n, b]`` is a per-lane scalar and the stage needs no data movement.  Nothing of size
(samples x segments x channels) is ever formed.

Two directions per configuration: 0 = forward (out rows <- input1 rows), 1 = gradient w.r.t. input1
(input1 rows <- grad_out rows, same coefficients, transposed weight).
"""
from __future__ import annotations

import os
from collections import OrderedDict

from .._tables import fingerprint, tp_coo
from ..irreps import Irreps, irrep_segments
from ..utils import tp_infos
from .gen_uvu import _lit, _sh, table_arrays

HERE = os.path.dirname(os.path.abspath(__file__))

CONFIGS = OrderedDict([
    ("sh1", (_sh(1), _sh(1), _sh(1), {})),
    ("sh2", (_sh(2), _sh(2), _sh(2), {})),
    ("sh3", (_sh(3), _sh(3), _sh(3), {})),
    # second operand = the scalar 1: channel mixing per irrep (IrrepsLinear between equal irreps)
    ("lin_sh2", (_sh(2), _sh(2), "0e", {})),
    ("lin_sh3", (_sh(3), _sh(3), "0e", {})),
])


def emit_direction(name: str, direction: int, coo, seg_out, seg_in1, gy: bool = False) -> str:
    """Body of one configuration.  ``gy``: instead of accumulating output rows, contract every tile with the rows of
    a second channelled operand ``g`` (the output gradient) into the gradient w.r.t. the harmonics,
    ``gy[b] += coef * sum_w g[m, w] * Z[w]`` (forward tables only)."""
    if direction == 0:
        out_idx, in_idx, blocks, din, dout = coo.M, coo.M1, seg_out, coo.D1, coo.DO
    else:
        out_idx, in_idx, blocks, din, dout = coo.M1, coo.M, seg_in1, coo.DO, coo.D1
    T = coo.coef.shape[0]
    # tiles in execution order: output irrep by output irrep (an output row is live only while its block runs),
    # inside a block path by path; tile = (path, input row) -> [(out row, y index, coef)]
    tiles, first_of_block, last_of_block, empty_rows = [], {}, {}, []
    for b0, b1 in zip(blocks[:-1], blocks[1:]):
        nnz = [t for t in range(T) if b0 <= out_idx[t] < b1]
        if not nnz:
            empty_rows += list(range(b0, b1))
            continue
        d = OrderedDict()
        for t in sorted(nnz, key=lambda t: (coo.p[t], in_idx[t], out_idx[t], coo.M2[t])):
            d.setdefault((int(coo.p[t]), int(in_idx[t])), []).append((int(out_idx[t]), int(coo.M2[t]), coo.coef[t]))
        first_of_block[len(tiles)] = list(range(b0, b1))
        tiles += list(d.items())
        last_of_block[len(tiles) - 1] = list(range(b0, b1))
    # weight fragments live in a ring of three buffers, fetched two path-runs ahead of their first use
    runs = []  # (path, first tile)
    for k, ((p, _), _) in enumerate(tiles):
        if not runs or runs[-1][0] != p or k in first_of_block:
            runs.append((p, k))
    run_of_tile = {}
    for j, (p, k0) in enumerate(runs):
        k1 = runs[j + 1][1] if j + 1 < len(runs) else len(tiles)
        for k in range(k0, k1):
            run_of_tile[k] = j
    L = []
    a = L.append
    a(f"struct UV_{name}_{'gy' if gy else 'd' + str(direction)} {{")
    a(f"  static constexpr int DIN = {din}, DOUT = {dout}, D2 = {coo.D2}, P = {coo.P};")
    a("  // xs: this lane's base into the staged input tile (row a of the sample at byte a * CIN * 2);")
    a("  // load_a(p, frag): fetch the weight fragments of path p;")
    if gy:
        a("  // load_g(row, t0, t1): this lane's 8 channels of row `row` of g; y receives this lane's partial sums.")
        a("  template <int CIN, class LoadA, class LoadG>")
        a("  __device__ __forceinline__ static void run(const unsigned char* xs, LoadA&& load_a, float (&y)[D2],")
        a("                                             LoadG&& load_g) {")
    else:
        a("  // store(row, t0, t1): emit one finished output row.")
        a("  template <int CIN, class LoadA, class Store>")
        a("  __device__ __forceinline__ static void run(const unsigned char* xs, LoadA&& load_a, const float (&y)[D2],")
        a("                                             Store&& store) {")
    a("    constexpr int KS = CIN / 32;")
    a("    bf16x8 w0[2][KS], w1[2][KS], w2[2][KS], b0[KS], b1[KS];")
    a("    floatx4 za0, za1, zb0, zb1;")
    a("    float yy[D2];")
    a("    for (int j = 0; j < D2; ++j) yy[j] = " + ("0.f;" if gy else "y[j];"))
    if empty_rows and not gy:
        a("    {")
        a("      floatx4 zero = {0};")
        for r in empty_rows:
            a(f"      store({r}, zero, zero);")
        a("    }")

    def load_b(k):
        a(f"    load_b<KS>(b{k % 2}, xs + {tiles[k][0][1]} * CIN * 2);")

    def chain(k):
        z = "za" if k % 2 == 0 else "zb"
        a(f"    mfma_chain<KS>(w{run_of_tile[k] % 3}, b{k % 2}, {z}0, {z}1);")
        j = run_of_tile[k]
        if runs[j][1] == k and j + 2 < len(runs):
            a(f"    load_a({runs[j + 2][0]}, w{(j + 2) % 3});")

    if tiles:
        a(f"    load_a({runs[0][0]}, w0);")
        if len(runs) > 1:
            a(f"    load_a({runs[1][0]}, w1);")
        load_b(0)
        if len(tiles) > 1:
            load_b(1)
        chain(0)
        a("    __builtin_amdgcn_sched_barrier(0);")
    for k, (key, terms) in enumerate(tiles):
        # slot k: fetch the input fragments of tile k+2, run the MFMA chain of tile k+1, and apply the Clebsch-Gordan
        # coefficients to tile k, whose chain ran in the previous slot
        if k in first_of_block:
            for r in first_of_block[k]:
                if gy:
                    a(f"    floatx4 o{r}_0, o{r}_1; load_g({r}, o{r}_0, o{r}_1);")
                else:
                    a(f"    floatx4 o{r}_0 = {{0}}, o{r}_1 = {{0}};")
        if k + 1 < len(tiles):
            chain(k + 1)
        if k + 2 < len(tiles):
            load_b(k + 2)
        cur = "za" if k % 2 == 0 else "zb"
        if gy:
            for (o, m2, c) in terms:
                a(f"    yy[{m2}] += {_lit(c)} * dot8(o{o}_0, o{o}_1, {cur}0, {cur}1);")
            # pin the partial sums (see the accumulators of the forward body)
            a("    asm volatile(\"\" : " + ", ".join(f'"+v"(yy[{m}])' for m in sorted({m2 for _, m2, _ in terms})) + ");")
            a("    __builtin_amdgcn_sched_barrier(0);")
            continue
        # hide the harmonics behind an empty asm per tile: equal (coefficient, harmonic) products recur in many
        # tiles and would otherwise be computed once and kept in registers across the whole body
        a("    " + " ".join(f'asm volatile("" : "+v"(yy[{m}]));' for m in sorted({m2 for _, m2, _ in terms})))
        # one update per output row: the harmonics that couple the same (output row, input row) pair are summed first
        by_row = OrderedDict()
        for (o, m2, c) in terms:
            by_row.setdefault(o, []).append((m2, c))
        for o, pairs in by_row.items():
            s_expr = " + ".join(f"{_lit(c)} * yy[{m2}]" for m2, c in pairs)
            a(f"    {{ const float s = {s_expr}; o{o}_0 += s * {cur}0; o{o}_1 += s * {cur}1; }}")
        # pin the updated accumulators: an output row is read again only when it is stored, and without this the
        # optimiser sinks every update of a block to its end, keeping all the block's tiles alive until then
        touched = sorted({o for o, _, _ in terms})
        a("    asm volatile(\"\" : " + ", ".join(f'"+v"(o{o}_0), "+v"(o{o}_1)' for o in touched) + ");")
        # the scheduler may interleave the MFMA chain above with these FMAs, but nothing crosses this point
        a("    __builtin_amdgcn_sched_barrier(0);")
        if k in last_of_block:
            for r in last_of_block[k]:
                a(f"    store({r}, o{r}_0, o{r}_1);")
    if gy:
        a("    for (int j = 0; j < D2; ++j) y[j] = yy[j];")
    a("  }")
    a("};")
    return "\n".join(L)


def emit_gw(name: str, coo, seg_out, seg_in1) -> str:
    """Per-path Clebsch-Gordan mixing for the weight gradient: ``G[a] = sum_(m,b) coef * y[b] * g[m]`` for every
    input row ``a`` the path reads, on 8-channel fp32 vectors (the matrix cores then contract ``x[a]`` with ``G[a]``
    over the samples)."""
    T = coo.coef.shape[0]
    L = []
    w = L.append
    a0, na, m0, nm = [], [], [], []
    for p in range(coo.P):
        for col, first, count in ((coo.M1, a0, na), (coo.M, m0, nm)):
            rows = sorted({int(col[t]) for t in range(T) if coo.p[t] == p})
            assert rows == list(range(rows[0], rows[0] + len(rows)))
            first.append(rows[0])
            count.append(len(rows))
    w(f"struct UV_{name}_gw {{")
    w(f"  static constexpr int D1 = {coo.D1}, DO = {coo.DO}, D2 = {coo.D2}, P = {coo.P}, MAX_ROWS = {max(na + nm)};")
    w("  // rows of the channelled input read by every path: first row and count")
    w(f"  static constexpr unsigned char A0[P] = {{{', '.join(map(str, a0))}}};")
    w(f"  static constexpr unsigned char NA[P] = {{{', '.join(map(str, na))}}};")
    w("  // rows of g (the output irrep) of every path: first row and count")
    w(f"  static constexpr unsigned char M0[P] = {{{', '.join(map(str, m0))}}};")
    w(f"  static constexpr unsigned char NM[P] = {{{', '.join(map(str, nm))}}};")
    w("  // src(h, j): 8 channels (pass h of 2) of row M0[p] + j of g as floats; dst(h, r, v): the mixed row for input row")
    w("  // A0[p] + r.  Both passes of a path sit in one case so that the coef * y products are formed once per path")
    w("  // and only for the path at hand.")
    w("  template <class Src, class Dst>")
    w("  __device__ __forceinline__ static void mix(int p, const float (&y)[D2], Src&& src, Dst&& dst) {")
    w("    switch (p) {")
    for p in range(coo.P):
        nnz = [t for t in range(T) if coo.p[t] == p]
        w(f"      case {p}: {{")
        prods = OrderedDict()
        for t in nnz:
            prods.setdefault((int(coo.M2[t]), _lit(coo.coef[t])), len(prods))
        for (b, c), i in prods.items():
            w(f"        const float s{i} = {c} * y[{b}];")
        for h in (0, 1):
            w("        {")
            for m in sorted({int(coo.M[t]) for t in nnz}):
                w(f"          const floatx8 g{m} = src({h}, {m - m0[p]});")
            for r in range(na[p]):
                terms = sorted((int(coo.M[t]), int(coo.M2[t]), _lit(coo.coef[t])) for t in nnz if coo.M1[t] == a0[p] + r)
                expr = " + ".join(f"s{prods[(b, c)]} * g{m}" for m, b, c in terms)
                w(f"          dst({h}, {r}, {expr});")
            w("        }")
        w("      } break;")
    w("      default: break;")
    w("    }")
    w("  }")
    w("};")
    return "\n".join(L)


def main(out_dir: str = None) -> str:
    out_dir = out_dir or os.path.join(HERE, "generated")
    os.makedirs(out_dir, exist_ok=True)
    chunks = ["// Generated by equitorch_amd/csrc/gen_uv.py; do not edit.", ""]
    entries = []
    for name, (io, i1, i2, kw) in CONFIGS.items():
        coo = tp_coo(tp_infos(Irreps(io), Irreps(i1), Irreps(i2), **kw)[0])
        seg_out, seg_in1 = irrep_segments(Irreps(io)), irrep_segments(Irreps(i1))
        chunks.append(f"// {name}: {i1} x {i2} -> {io}")
        for d in (0, 1):
            chunks.append(emit_direction(name, d, coo, seg_out, seg_in1))
        chunks.append(emit_direction(name, 0, coo, seg_out, seg_in1, gy=True))
        chunks.append(emit_gw(name, coo, seg_out, seg_in1))
        chunks.append("\n".join([f"struct UV_{name}_tab {{",
                                 f"  static constexpr int D1 = {coo.D1}, D2 = {coo.D2}, DO = {coo.DO}, P = {coo.P}, "
                                 f"NNZ = {coo.coef.shape[0]};", *table_arrays(coo), "};"]))
        entries.append((name, fingerprint(coo), fingerprint(coo, "bf16"), fingerprint(coo, "f16")))
        chunks.append("")
    chunks.append("#define CGTP_FOREACH_UV_CONFIG(X) \\")
    chunks.append(" \\\n".join(f"  X(UV_{n}_d0, UV_{n}_d1, UV_{n}_gy, UV_{n}_gw, UV_{n}_tab, 0x{fp:016x}ull, 0x{fb:016x}ull, 0x{fh:016x}ull, \"{n}\")"
                              for n, fp, fb, fh in entries))
    chunks.append("")
    path = os.path.join(out_dir, "uv_configs.inc")
    text = "\n".join(chunks)
    if not os.path.exists(path) or open(path).read() != text:
        with open(path, "w") as f:
            f.write(text)
    return path


if __name__ == "__main__":
    print(main())
