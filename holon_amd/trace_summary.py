"""Per-kernel times out of a `rocprofv3 --kernel-trace` database of a bench.py or CLI run.

    python -m holon_amd.trace_summary DB                 every kernel of the run, summed by name
    python -m holon_amd.trace_summary DB --step decode   one decode step (the one before the last embedding kernel)
    python -m holon_amd.trace_summary DB --step prefill  the third step of the run (bench.py's last timed prompt step)
    ... --classes                                        after the kernels, the step's time by class of kernel:
                                                         attention, matrix products, elementwise, sampling, other

A step is what lies between two embedding kernels: every step of the engine starts with one. The database is the
`*_results.db` file that rocprofv3 writes (SQLite: `rocpd_kernel_dispatch` joined with `rocpd_info_kernel_symbol`).
"""
from __future__ import annotations

import argparse
import collections
import sqlite3

SHORT = (("_Z18gemm_skinny_kernelILi", "gemm_skinny<"), ("_Z22gemm_skinny_glu_kernelILi", "gemm_skinny_glu<"),
         ("_Z18rmsnorm_row_kernelI", "rmsnorm_row<"), ("_Z30qk_norm_rope_write_fast_kernelI", "qk_norm_rope_write_fast<"),
         ("_Z18attn_decode_kernelILi", "attn_decode<"), ("_Z19attn_prefill_kernelILi", "attn_prefill<"),
         ("_Z24attn_prefill_wide_kernelILi", "attn_prefill_wide<"), ("_Z23attn_prefill_lds_kernelILi", "attn_prefill_lds<"),
         ("_Z23attn_prefill_dma_kernel8AttnArgs", "attn_prefill_dma"), ("_Z24attn_prefill_pair_kernelILi", "attn_prefill_pair<"),
         ("_Z17attn_merge_kernel", "attn_merge"), ("_Z13argmax_kernel", "argmax"), ("_Z20argmax_pieces_kernel", "argmax_pieces"),
         ("_Z23argmax_of_pieces_kernel", "argmax_of_pieces"), ("_Z16embedding_kernel", "embedding"),
         ("_Z15gemm_f32_kernel", "gemm_f32"), ("_Z13sample_kernel", "sample"),
         ("_ZN12_GLOBAL__N_116gemm_rows_kernelILi", "gemm_rows<"),
         ("_Z19silu_mul_vec_kernel", "silu_mul_vec"), ("Cijk_Alik_Bljk_BBS_BH_Bias_HA_S_SAV_UserArgs_", "hipBLASLt "),
         ("Custom_Cijk_Alik_Bljk_BBS_BH_Bias_HA_S_SAV_NTD_SK3_UserArgs_", "hipBLASLt custom "))


def short_name(name: str) -> str:
    name = name.split("(")[0]
    for long, brief in SHORT:
        if name.startswith(long):
            name = brief + name[len(long):]
    return name[:64]


def dispatches(path: str) -> list[tuple]:
    """(name, start ns, end ns, blocks x, y, z) of every kernel, in start order."""
    db = sqlite3.connect(path)
    rows = db.execute(
        "select s.kernel_name, d.start, d.end, d.grid_size_x, d.grid_size_y, d.grid_size_z, d.workgroup_size_x "
        "from rocpd_kernel_dispatch d join rocpd_info_kernel_symbol s on d.kernel_id = s.id order by d.start").fetchall()
    return [(n, st, en, gx // max(wx, 1), gy, gz) for n, st, en, gx, gy, gz, wx in rows]


CLASSES = (("attention", ("attn_",)), ("matrix products", ("gemm_", "Cijk_", "Custom_Cijk_", "hipBLASLt")),
           ("elementwise", ("rmsnorm", "silu_mul", "qk_norm_rope", "v_write", "kv_write", "embedding", "sum_parts",
                            "row_sumsq", "scatter_rows")),
           ("sampling", ("argmax", "sample_kernel", "store_tokens", "logprobs")))


def kernel_class(name: str) -> str:
    for label, marks in CLASSES:
        if any(mark in name for mark in marks):
            return label
    return "other (copies, library elementwise)"


def by_class(rows: list[tuple]) -> str:
    """The step's kernel time by class of kernel, as a share of the time from its first start to its last end (what
    no kernel covers is the gaps between kernels)."""
    span = (rows[-1][2] - rows[0][1]) / 1e3
    took: dict[str, float] = collections.OrderedDict()
    for name, st, en, *_ in rows:
        took[kernel_class(name)] = took.get(kernel_class(name), 0.0) + (en - st) / 1e3
    out = [f"{'us':>10} {'of step':>8}  class"]
    for label, us in sorted(took.items(), key=lambda kv: -kv[1]):
        out.append(f"{us:10.1f} {100 * us / span:7.1f}%  {label}")
    out.append(f"{span - sum(took.values()):10.1f} {100 * (span - sum(took.values())) / span:7.1f}%  between kernels")
    return "\n".join(out)


def summarise(rows: list[tuple], title: str, top: int, with_grid: bool) -> str:
    agg: dict[str, list] = collections.OrderedDict()
    total = 0.0
    for name, st, en, gx, gy, gz in rows:
        key = short_name(name) + (f"  grid {gx}x{gy}x{gz}" if with_grid else "")
        a = agg.setdefault(key, [0, 0.0])
        a[0] += 1
        a[1] += (en - st) / 1e3
        total += (en - st) / 1e3
    out = [f"{title}: {len(rows)} kernels, {total / 1e3:.3f} ms of kernel time, "
           f"{(rows[-1][2] - rows[0][1]) / 1e6:.3f} ms first start to last end",
           f"{'total us':>10} {'share':>6} {'calls':>6} {'avg us':>8}  kernel"]
    for key, (calls, us) in sorted(agg.items(), key=lambda kv: -kv[1][1])[:top]:
        out.append(f"{us:10.1f} {100 * us / total:5.1f}% {calls:6d} {us / calls:8.1f}  {key}")
    return "\n".join(out)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("db")
    ap.add_argument("--step", choices=("decode", "prefill"), help="one step instead of the whole run")
    ap.add_argument("--index", type=int, default=2, help="which step of the run --step prefill takes (default: the third)")
    ap.add_argument("--top", type=int, default=16)
    ap.add_argument("--classes", action="store_true", help="also the time by class of kernel")
    args = ap.parse_args(argv)
    rows = dispatches(args.db)
    if not rows:
        print("no kernel dispatches in this database")
        return 1
    starts = [i for i, r in enumerate(rows) if "embedding_kernel" in r[0]]
    if args.step == "decode":
        if len(starts) < 3:
            print("fewer than three steps in this trace")
            return 1
        rows = rows[starts[-3]:starts[-2]]
        print(summarise(rows, "one decode step", args.top, True))
    elif args.step == "prefill":
        if len(starts) < args.index + 2:
            print(f"fewer than {args.index + 2} steps in this trace")
            return 1
        rows = rows[starts[args.index]:starts[args.index + 1]]
        print(summarise(rows, "one prompt step", args.top, True))
    else:
        print(summarise(rows, "whole run", args.top, False))
    if args.classes:
        print(by_class(rows))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
