"""The reference's sweep over datasets x train-mask ratios x model depths (EPPGCN/bench_EPPGCN.py:17-61)
over this package's driver, in one process.

    python -m eppgcn_amd.bench_eppgcn [--groupsize_model regression_equation|SAGPG|fixed_value]
                                      [--dataRoot DIR] [--datasets NAME[,DIM,CLASSES] ...]
                                      [--ratios R ...] [--layers L ...] [--hidden H ...]
                                      [--num_epoches E] [--loadFromTxt True|False]

Per combination it runs ``eppgcn_amd.gcn_main.main`` with the flags the reference's script formats
(EPPGCN/bench_EPPGCN.py:54-59) - so the driver prints its usual report (``||dataset ratio layers``,
per-kernel times, ``for_time`` ... ``Time``) - and then one JSON line with the same figures.  The
defaults are the reference's: its ten datasets with their feature widths and class counts, ratios
0.1 / 0.3 / 0.5 / 0.8, depths 3-6, hidden width 16, group sizes from the fitted regression
(``regression_equation`` = ``--backsize_mode map``; ``fixed_value`` = constant 32; ``SAGPG`` needs
predictor weights the reference does not publish and is refused by the driver).

Differences, all deliberate: the runs share one process instead of one ``os.system`` call each (the
execution-plan cache of the extension module is cleared between them); the data root is a flag
(``<dataRoot>/<dataset>/`` holds ``<dataset>_snap`` or ``<dataset>.npz`` and the mask files) where the
reference hard-codes the authors' directory; a dataset whose files are missing is reported and
skipped; a dataset name may also be a synthetic graph of ``eppgcn_amd.graphs.make_graph``.
"""
from __future__ import annotations

import argparse
import json
import os.path as osp
import sys

# (name, feature width, classes), EPPGCN/bench_EPPGCN.py:17-31
REFERENCE_DATASETS = [
    ("cora", 1433, 7), ("citeseer", 3703, 6), ("pubmed", 500, 3), ("youtube", 64, 47), ("amazon", 96, 22),
    ("corafull", 64, 32), ("catalog", 64, 32), ("twitter", 64, 32), ("google", 64, 32), ("dblp", 64, 32),
]
REFERENCE_RATIOS = [0.1, 0.3, 0.5, 0.8]
REFERENCE_LAYERS = [3, 4, 5, 6]
BACK_MODES = {"regression_equation": ("map", 0), "SAGPG": ("net", 0), "fixed_value": ("constant", 32)}


def parse_dataset(text: str):
    """``name`` (feature width 96, 22 classes, or the reference's figures for its own datasets) or
    ``name,dim,classes``."""
    parts = text.split(",")
    if len(parts) == 3:
        return parts[0], int(parts[1]), int(parts[2])
    if len(parts) != 1:
        raise argparse.ArgumentTypeError(f"'{text}': expected NAME or NAME,DIM,CLASSES")
    for name, dim, classes in REFERENCE_DATASETS:
        if name == text:
            return name, dim, classes
    return text, 96, 22


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(description="datasets x train ratios x depths sweep over eppgcn_amd.gcn_main")
    ap.add_argument("--groupsize_model", type=str, default="regression_equation", choices=sorted(BACK_MODES))
    ap.add_argument("--dataRoot", type=str, default="../osdi-ae-graphs", help="directory with one folder per dataset")
    ap.add_argument("--datasets", type=parse_dataset, nargs="+", default=list(REFERENCE_DATASETS))
    ap.add_argument("--ratios", type=float, nargs="+", default=REFERENCE_RATIOS)
    ap.add_argument("--layers", type=int, nargs="+", default=REFERENCE_LAYERS)
    ap.add_argument("--hidden", type=int, nargs="+", default=[16])
    ap.add_argument("--num_epoches", type=int, default=100)
    ap.add_argument("--loadFromTxt", type=str, default="True", choices=["True", "False"])
    ap.add_argument("--degree_norm", type=str, default="sqrt", choices=["sqrt", "inv_sqrt"])
    ap.add_argument("--with_unpruned", action="store_true",
                    help="run every combination a second time with the unpruned backward aggregation (the driver's "
                         "--prune False) and report its times beside the pruned ones")
    return ap


def driver_arguments(args, name, dim, classes, hidden, ratio, layers, prune=True):
    """The flags of EPPGCN/bench_EPPGCN.py:54-59 for one combination."""
    back_mode, backsize = BACK_MODES[args.groupsize_model]
    folder = osp.join(args.dataRoot, name)
    return ["--dataset", name, "--dim", str(dim), "--hidden", str(hidden), "--classes", str(classes),
            "--layers", str(layers), "--partSize", "0", "--model", "gcn", "--warpPerBlock", "8",
            "--manual_mode", "False", "--verbose_mode", "False", "--loadFromTxt", args.loadFromTxt,
            "--dataDir", folder if osp.isdir(folder) else args.dataRoot, "--train_ratio", str(ratio),
            "--backsize_mode", back_mode, "--backsize", str(backsize), "--num_epoches", str(args.num_epoches),
            "--degree_norm", args.degree_norm, "--prune", str(bool(prune))]


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    import torch

    from . import gcn_main, gnnadvisor
    GNNA = gnnadvisor()
    failures = 0
    for hidden in args.hidden:
        for name, dim, classes in args.datasets:
            for ratio in args.ratios:
                for layers in args.layers:
                    line = {"dataset": name, "dim": dim, "classes": classes, "hidden": hidden, "train_ratio": ratio,
                            "layers": layers, "groupsize_model": args.groupsize_model}
                    report = {}
                    try:
                        rc = gcn_main.main(driver_arguments(args, name, dim, classes, hidden, ratio, layers), report)
                        line.update(report, status="ok" if rc == 0 else f"driver returned {rc}")
                        if rc == 0 and args.with_unpruned:
                            GNNA.clear_plans()
                            plain = {}
                            rc = gcn_main.main(driver_arguments(args, name, dim, classes, hidden, ratio, layers, False), plain)
                            line["unpruned"] = {k: plain.get(k) for k in ("Time", "for_time", "back_time", "back_agg_time",
                                                                          "for_agg_time", "build_time")}
                    except FileNotFoundError as exc:
                        rc = 0
                        line.update(status="skipped", reason=str(exc))
                    failures += rc != 0
                    print(json.dumps(line), flush=True)
                    GNNA.clear_plans()          # the next combination has other group arrays
                    torch.cuda.empty_cache()
    return 1 if failures else 0


if __name__ == "__main__":
    sys.exit(main())
