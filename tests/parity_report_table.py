"""Turns the JSON lines that the full-size GPU tests append to $H2O4GPU_PARITY_REPORT
(tests/test_gpu_configs.py, tests/test_gpu_entry_points_full_size.py) into the markdown tables of
the parity summary. Numbers only; nothing here touches a GPU.

    python tests/parity_report_table.py parity_report.jsonl
"""
import json
import sys


def _f(v, fmt="%.1e"):
    return "-" if v is None else (fmt % v)


def main(path):
    full, entry, mind = [], [], []
    for line in open(path):
        r = json.loads(line)
        if "lockstep_start" in r:
            full.append(r)
        elif r.get("kind") == "entry_points":
            entry.append(r)
        elif r.get("kind") == "min_distance_error":
            mind.append(r)
    out = []
    out.append("### Lock-step on all rows (one assignment pass from the same centroids)\n")
    out.append("Mismatches against the oracle: total (excused by the 1e-5 gap / by the rounding floor), worst "
               "relative gap; in brackets the oracle against itself with the features summed in descending "
               "order, same columns.\n")
    out.append("| Config | kernel | at the start | at the fitted centroids | keys vs exact compare: flips start / fitted |")
    out.append("|---|---|---|---|---|")

    def cell(s):
        return "%d (%d / %d), %s [%d (%d / %d), %s]" % (
            s["mismatch"], s["excused_by_gap"], s["excused_by_noise_floor"], _f(s["worst_gap"]),
            s["oracle_desc_vs_asc_mismatch"], s.get("oracle_desc_vs_asc_excused_by_gap", -1),
            s.get("oracle_desc_vs_asc_excused_by_noise_floor", -1), _f(s["oracle_desc_vs_asc_worst_gap"]))

    for r in full:
        a, b = r["lockstep_start"], r["lockstep_fitted"]
        flips = "-"
        if "keys_vs_exact_compare_flips" in a:
            flips = "%d / %d" % (a["keys_vs_exact_compare_flips"], b["keys_vs_exact_compare_flips"])
        out.append("| %s %s | %s | %s | %s | %s |" % (r["config"], r["dtype"], r["variant"], cell(a), cell(b), flips))
    out.append("")
    out.append("### End to end from the same start, fixed iteration count, all rows\n")
    out.append("| Config | iterations compared | centroid error | label differences | objective, relative | "
               "same three for the oracle against itself (descending order) | engine with the exact compare: "
               "centroid error |")
    out.append("|---|---|---|---|---|---|---|")
    for r in full:
        e = r["end_to_end"]
        out.append("| %s %s | %d of %d | %s | %d | %s | %s, %d, %s | %s |" % (
            r["config"], r["dtype"], e["iterations"], r["fit_iterations"], _f(e["centroid_err"]),
            e["label_diffs"], _f(e["inertia_rel_diff"]), _f(e["oracle_desc_vs_asc_centroid_err"]),
            e["oracle_desc_vs_asc_label_diffs"], _f(e["oracle_desc_vs_asc_inertia_rel_diff"]),
            _f(e.get("exact_compare_centroid_err"))))
    out.append("")
    out.append("### The reference's four symbols at full size\n")
    out.append("| Config | rows | iterations | fit through make_ptr_*_kmeans equals the handle-level fit | "
               "predict (dopredict = 1) on all rows equals labels | transform vs the oracle, worst element |")
    out.append("|---|---|---|---|---|---|")
    for r in entry:
        t = "-"
        if "transform_elements" in r:
            t = "%d elements, %.1f eps (xx + cc) (bar %.0f)" % (
                r["transform_elements"], r["transform_worst_err_in_eps_xx_cc"], r["transform_bar_in_eps_xx_cc"])
        out.append("| %s %s | %d | %d | bit for bit | %d of %d | %s |" % (
            r["config"], r["dtype"], r["n"], r["iterations"], r["predict_rows"], r["n"], t))
    out.append("")
    out.append("### Error of the minimum distance against float64, in units of eps (|x|^2 + |c|^2)\n")
    out.append("| Config (20,000 rows) | kernel | engine: mean, rms, max | oracle, ascending | oracle, descending |")
    out.append("|---|---|---|---|---|")
    for r in mind:
        def c(x):
            return "%+.3f, %.2f, %.1f" % (x["mean"], x["rms"], x["max_abs"])
        out.append("| %s d = %d, k = %d | %s | %s | %s | %s |" % (
            r["config"], r["d"], r["k"], r["variant"], c(r["engine"]), c(r["oracle_ascending"]),
            c(r["oracle_descending"])))
    print("\n".join(out))


if __name__ == "__main__":
    if len(sys.argv) != 2:
        sys.exit("usage: python tests/parity_report_table.py <file the tests wrote to $H2O4GPU_PARITY_REPORT>")
    main(sys.argv[1])
