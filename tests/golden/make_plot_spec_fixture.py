"""Writes tests/golden/plot_spec_series.json: the `regex:` strings (and their series labels) of the
reference's figure specifications, figures/spec/*.yml, which select benchmark names from the JSON
the harness writes, and the names of the JSON fields every figure plots (xaxis.field, yaxis.field and
their scales).  Data only: strings and numbers copied from YAML values, no code of the reference.

Run in the container that holds the reference:  python tests/golden/make_plot_spec_fixture.py [/root/reference]
"""
import json
import os
import sys

import yaml

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    spec_dir = os.path.join(ref, "figures", "spec")
    out = {}
    for name in sorted(os.listdir(spec_dir)):
        if not name.endswith(".yml"):
            continue
        with open(os.path.join(spec_dir, name)) as f:
            doc = yaml.load(f, Loader=yaml.SafeLoader)
        series = []
        for s in (doc or {}).get("series") or []:
            if isinstance(s, dict) and "regex" in s:
                entry = {"label": str(s.get("label", "")), "regex": str(s["regex"])}
                for k in ("xfield", "yfield"):
                    if k in s:
                        entry[k] = str(s[k])
                series.append(entry)
        axes = {}
        for axis in ("xaxis", "yaxis"):
            a = (doc or {}).get(axis) or {}
            axes[axis] = {"field": str(a.get("field", "real_time")), "scale": str(a.get("scale", 1.0))}
        out[name] = {"input_file": os.path.basename(str((doc or {}).get("input_file", ""))), "series": series, **axes}
    path = os.path.join(HERE, "plot_spec_series.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
        f.write("\n")
    print(f"{path}: {len(out)} specs, {sum(len(v['series']) for v in out.values())} series")


if __name__ == "__main__":
    main()
