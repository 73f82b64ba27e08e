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

import numpy as np

from .._tables import fingerprint, tp_coo
from ..irreps import Irreps, irrep_segments
from ..utils import tp_infos
from .gen_uvu import _lit, _sh

HERE = os.path.dirname(os.path.abspath(__file__))

CONFIGS = OrderedDict([
    ("sh1", (_sh(1), _sh(1), _sh(1), {})),
    ("sh2", (_sh(2), _sh(2), _sh(2), {})),
    ("sh3", (_sh(3), _sh(3), _sh(3), {})),
])


def emit_direction(name: str, direction: int, coo, seg_out, seg_in1) -> str:
    if direction == 0:
        out_idx, in_idx, blocks, din, dout = coo.M, coo.M1, seg_out, coo.D1, coo.DO
    else:
        out_idx, in_idx, blocks, din, dout = coo.M1, coo.M, seg_in1, coo.DO, coo.D1
    T = coo.coef.shape[0]
    L = []
    a = L.append
    a(f"struct UV_{name}_d{direction} {{")
    a(f"  static constexpr int DIN = {din}, DOUT = {dout}, D2 = {coo.D2}, P = {coo.P};")
    a("  // xs: this lane's base into the staged input tile (row a of the sample at byte a * CIN * 2);")
    a("  // load_a(p, frag): fetch the weight fragments of path p; store(row, tile): emit one finished output row.")
    a("  template <int CIN, class LoadA, class Store>")
    a("  __device__ __forceinline__ static void run(const unsigned char* xs, LoadA&& load_a, const float (&y)[D2],")
    a("                                             Store&& store) {")
    a("    constexpr int KS = CIN / 32;")
    a("    bf16x8 wa[2][KS], wb[2][KS];")
    a("    floatx4 za0, za1, zb0, zb1;")
    a("    float yy[D2];")
    a("    for (int j = 0; j < D2; ++j) yy[j] = y[j];")
    for b0, b1 in zip(blocks[:-1], blocks[1:]):
        rows = list(range(b0, b1))
        nnz = [t for t in range(T) if b0 <= out_idx[t] < b1]
        if not nnz:
            a("    {")
            a("      floatx4 zero = {0};")
            for r in rows:
                a(f"      store({r}, zero, zero);")
            a("    }")
            continue
        # tiles of this block: (path, input row) -> [(out row, y index, coef)]
        tiles = OrderedDict()
        for t in sorted(nnz, key=lambda t: (coo.p[t], in_idx[t], out_idx[t], coo.M2[t])):
            tiles.setdefault((int(coo.p[t]), int(in_idx[t])), []).append((int(out_idx[t]), int(coo.M2[t]), coo.coef[t]))
        keys = list(tiles)
        paths = list(OrderedDict.fromkeys(p for p, _ in keys))
        a("    {")
        for r in rows:
            a(f"      floatx4 o{r}_0 = {{0}}, o{r}_1 = {{0}};")
        a(f"      load_a({paths[0]}, wa);")
        # software pipeline: the MFMA chain of tile k+1 is issued before the FMAs that consume tile k
        def chain(dst, key):
            p, row = key
            frag = "wa" if paths.index(p) % 2 == 0 else "wb"
            a(f"      mfma_chain<KS>({frag}, xs + {row} * CIN * 2, {dst}0, {dst}1);")
        prev_path = None
        for k, key in enumerate(keys):
            p = key[0]
            if p != prev_path:
                nxt = paths.index(p) + 1
                if nxt < len(paths):
                    a(f"      load_a({paths[nxt]}, {'wa' if nxt % 2 == 0 else 'wb'});")
                prev_path = p
            if k == 0:
                chain("za", key)
            cur = "za" if k % 2 == 0 else "zb"
            if k + 1 < len(keys):
                # weight fragments of the next tile's path were requested one path earlier
                chain("zb" if k % 2 == 0 else "za", keys[k + 1])
            # hide the harmonics behind an empty asm per tile: equal (coefficient, harmonic) products recur in many
            # tiles and would otherwise be computed once and kept in registers across the whole body
            a("      " + " ".join(f'asm volatile("" : "+v"(yy[{m}]));' for m in sorted({m2 for _, m2, _ in tiles[key]})))
            for (o, m2, c) in tiles[key]:
                a(f"      {{ const float s = {_lit(c)} * yy[{m2}]; o{o}_0 += s * {cur}0; o{o}_1 += s * {cur}1; }}")
            # pin the updated accumulators: an output row is read again only when it is stored, and without this the
            # optimiser sinks every update of a block to its end, keeping all the block's tiles alive until then
            touched = sorted({o for o, _, _ in tiles[key]})
            a("      asm volatile(\"\" : " + ", ".join(f'"+v"(o{o}_0), "+v"(o{o}_1)' for o in touched) + ");")
            # the scheduler may interleave the MFMA chain above with these FMAs, but nothing crosses this point:
            # without it weight-fragment loads and whole chains are hoisted until thousands of registers are live
            a("      __builtin_amdgcn_sched_barrier(0);")
        for r in rows:
            a(f"      store({r}, o{r}_0, o{r}_1);")
        a("    }")
    a("  }")
    a("};")
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
        entries.append((name, fingerprint(coo)))
        chunks.append("")
    chunks.append("#define CGTP_FOREACH_UV_CONFIG(X) \\")
    chunks.append(" \\\n".join(f"  X(UV_{n}_d0, UV_{n}_d1, 0x{fp:016x}ull, \"{n}\")" for n, fp in entries))
    chunks.append("")
    path = os.path.join(out_dir, "uv_configs.inc")
    text = "\n".join(chunks)
    if not os.path.exists(path) or open(path).read() != text:
        with open(path, "w") as f:
            f.write(text)
    return path


if __name__ == "__main__":
    print(main())
