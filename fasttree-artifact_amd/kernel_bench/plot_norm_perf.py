"""Normalised-performance chart of the kernel sweep, in the manner of the reference's figure
(kernel_bench/plot_norm_perf.py, assets/results.png): one panel per head configuration, one group
of bars per tree, every engine's speed divided by the fastest engine's of that tree.

    python plot_norm_perf.py --input sweep/results.md --preset mi355x --output sweep/results.png

Reads the table ``run_benchmark.py`` writes (milliseconds per engine), so the engines are the
ones measured here: the gathered decode without sharing, the naive plan, DeFT-Flatten (its own
masked kernel), multi-level cascade attention, the tree decode without the greedy merge, and the
tree decode.
"""
import argparse

ENGINES = [("gathered ms", "Gathered (no sharing)", "#CCCCCC"),
           ("tree, naive ms", "Tree, naive", "#B4C7E7"),
           ("DeFT ms", "DeFT", "#FFE699"),
           ("cascade ms", "Cascade", "#F6CAE5"),
           ("tree, w/o greedy ms", "Tree w/o greedy", "#F8CBAD"),
           ("tree ms", "Tree decode", "#C5796A")]


def read_table(path, preset):
    """Rows of the sweep table as dicts keyed by the column titles, for one preset."""
    header, rows = None, []
    for line in open(path):
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if len(cells) < 8:
            continue
        if header is None:
            if cells[0].startswith("tree"):
                header = cells
            continue
        if set(cells[0]) <= set("-: "):
            continue
        row = dict(zip(header, cells))
        if row.get("preset") == preset:
            rows.append(row)
    if header is None:
        raise SystemExit(f"{path}: no sweep table found")
    return rows


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--input", required=True, help="results.md written by run_benchmark.py")
    ap.add_argument("--preset", default="mi355x")
    ap.add_argument("--output", default="results.png")
    args = ap.parse_args(argv)
    rows = read_table(args.input, args.preset)
    engines = [e for e in ENGINES if rows and e[0] in rows[0]]
    heads = []
    for r in rows:
        if r["q/kv heads"] not in heads:
            heads.append(r["q/kv heads"])

    import matplotlib
    matplotlib.use("Agg")
    import matplotlib.pyplot as plt

    fig, axes = plt.subplots(len(heads), 1, figsize=(16, 3.2 * len(heads)), sharex=True, squeeze=False)
    width = 1.0 / (len(engines) + 2)
    for ax, head in zip(axes[:, 0], heads):
        part = [r for r in rows if r["q/kv heads"] == head]
        for i, (column, label, colour) in enumerate(engines):
            speed = []
            for r in part:
                best = min(float(r[c]) for c, _, _ in engines)
                speed.append(best / float(r[column]))
            ax.bar([x + width * i for x in range(len(part))], speed, width=width, label=label, color=colour, edgecolor="k", linewidth=0.5)
        ax.set_ylim(0, 1.05)
        ax.set_ylabel(f"{head} heads\nnormalised speed")
        ax.set_xticks([x + width * (len(engines) - 1) / 2 for x in range(len(part))])
        ax.set_xticklabels([r[rows_key(r)].replace(" / ", "\n") for r in part], fontsize=7, rotation=30, ha="right")
        ax.grid(axis="y", linewidth=0.3)
    axes[0, 0].legend(ncol=len(engines), loc="lower center", bbox_to_anchor=(0.5, 1.02), frameon=False)
    fig.tight_layout()
    fig.savefig(args.output, dpi=130)
    print(f"wrote {args.output}: {len(rows)} cases, preset {args.preset}")
    return 0


def rows_key(row):
    return next(k for k in row if k.startswith("tree (nodes"))


if __name__ == "__main__":
    raise SystemExit(main())
