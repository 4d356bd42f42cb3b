"""Plots of the sweeps' JSON files, one PNG per sweep (log-scaled x axis, one line per
provider, the q10-q90 band shaded), in the manner of the reference's benchmark gallery
(scripts/plot_benchmark.py there).

    python -m benchmarks.plot <dir with the sweeps' JSON files> [output dir]
"""

from __future__ import annotations

import json
import sys
from pathlib import Path


def main():
    import matplotlib

    matplotlib.use("Agg")
    import matplotlib.pyplot as plt

    src = Path(sys.argv[1])
    dst = Path(sys.argv[2]) if len(sys.argv) > 2 else Path(__file__).with_name("plots")
    dst.mkdir(parents=True, exist_ok=True)
    for path in sorted(src.glob("*.json")):
        sweep = json.loads(path.read_text())
        rows = sweep["rows"]
        xs = [r["x"] for r in rows]
        fig, ax = plt.subplots(figsize=(5.2, 3.4), dpi=110)
        for provider in [k for k in rows[0] if k != "x"]:
            mid = [r[provider][0] for r in rows]
            lo = [min(r[provider][1:]) for r in rows]
            hi = [max(r[provider][1:]) for r in rows]
            (line,) = ax.plot(xs, mid, marker="o", markersize=3, linewidth=1.2, label=provider)
            ax.fill_between(xs, lo, hi, color=line.get_color(), alpha=0.15)
        ax.set_xscale("log", base=2)
        ax.set_xlabel(sweep["x"])
        ax.set_ylabel(sweep["unit"])
        ax.set_title(sweep["name"] + " - MI355X", fontsize=9)
        ax.grid(True, alpha=0.3)
        ax.legend(fontsize=7)
        fig.tight_layout()
        fig.savefig(dst / (path.stem + ".png"))
        plt.close(fig)
        print("wrote", dst / (path.stem + ".png"))


if __name__ == "__main__":
    main()
