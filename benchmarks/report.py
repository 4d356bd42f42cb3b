"""Turn the JSON files written by the sweeps into one markdown report.

    python -m benchmarks.report <dir with the sweeps' JSON files> [output.md]
"""

from __future__ import annotations

import json
import sys
from pathlib import Path

ORDER = ["lm2exp", "lt2exp", "vmax", "matmax", "mm", "vadd"]

HEADER = """# Reference benchmark grid on one MI355X

The sweeps of the reference (`benchmarks/lm2exp.py:26-56`, `benchmarks/lt2exp.py:32-63`, `benchmarks/max.py:16-66` there),
re-run with these kernels: same shapes, same input distributions (`rand` weights, `randn` log-values, seed 42),
same metrics (GB/s of input bytes for lm2exp / lt2exp; comparisons per second, labelled TFLOPS, for the max
reductions) and the same protocol (median of event-timed calls, each preceded by a 512 MiB cache flush).
`torch` is the reference's eager torch recipe on the same GPU (rocBLAS bmm + elementwise kernels); `triturus` is
this repository; `triturus (allow_tf32)` is the same call after `set_tf32_enabled(True)` (split-bf16 matrix path).  Run with
`python -m benchmarks.lm2exp|lt2exp|max|mm <dir>`, then `python -m benchmarks.report <dir>`.
"""


def stem(name: str) -> str:
    return "".join(c if c.isalnum() else "_" for c in name)


def table(sweep: dict) -> str:
    rows = sweep["rows"]
    providers = [k for k in rows[0] if k != "x"]
    ratio = "triturus" in providers and "torch" in providers
    head = [sweep["x"]] + providers + (["triturus / torch"] if ratio else [])
    lines = [f"## {sweep['name']}  [{sweep['unit']}]", "", "| " + " | ".join(head) + " |",
             "|" + "---:|" * len(head)]
    gbps = "GB/s" in sweep["unit"]
    for r in rows:
        cells = [str(r["x"])] + [f"{r[p][0]:.1f}" if gbps else f"{r[p][0]:.3g}" for p in providers]
        if ratio:
            cells.append(f"{r['triturus'][0] / r['torch'][0]:.2f}")
        lines.append("| " + " | ".join(cells) + " |")
    plot = Path(__file__).with_name("plots") / (stem(sweep["name"]) + ".png")
    if plot.exists():
        lines += ["", f"![{sweep['name']}](plots/{plot.name})"]
    return "\n".join(lines)


def main():
    src = Path(sys.argv[1])
    dst = Path(sys.argv[2]) if len(sys.argv) > 2 else Path(__file__).with_name("RESULTS.md")
    sweeps = [json.loads(p.read_text()) for p in sorted(src.glob("*.json"))]
    sweeps.sort(key=lambda s: (next((i for i, o in enumerate(ORDER) if s["name"].startswith(o)), 99), s["name"]))
    dst.write_text(HEADER + "\n" + "\n\n".join(table(s) for s in sweeps) + "\n")
    print(f"wrote {dst} ({len(sweeps)} sweeps)")


if __name__ == "__main__":
    main()
