"""Writes tests/golden/reference_tuner_keys.json: the problem keys (and the
rank-0 tile the reference's tuner stored for each) of every tuner cache the
reference ships under benchmark/**/tuner_cache.db.

The keys are data: `M_N_K_dtypeA_dtypeB_layoutA_layoutB[_seven epilogue counts]`
for GEMMs, `L_M_N_K_...` for batched ones (python/gtl/compiler/autotuner/
gemm_tuner.py:95-100, bmm_tuner.py, tuner_base.py:107-152), `(rows, columns)`
plus the counts for the softmax / layer norm anchors.  They are the reference's
own catalogue of the problems its code generator was run on, which
tests/test_reference_keys.py uses as a coverage checklist.  The sqlite files are
opened read-only; nothing of the reference is executed.

    python tests/golden/make_reference_tuner_keys.py     # in the build container (needs /root/reference)
"""
import glob
import json
import os
import sqlite3

REFERENCE = os.environ.get("EVT_REFERENCE_ROOT", "/root/reference")
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_tuner_keys.json")
TABLES = ("best_config_mm", "best_config_bmm", "best_config_softmax", "best_config_softmax_backward",
          "best_config_layernorm", "best_config_layernorm_backward")
SHORT = (("cutlass::half_t", "h"), ("cutlass::bfloat16_t", "bf"), ("cutlass::layout::RowMajor", "R"),
         ("cutlass::layout::ColumnMajor", "C"))


def main():
    tables = {t: {} for t in TABLES}
    files = sorted(glob.glob(os.path.join(REFERENCE, "benchmark", "**", "tuner_cache.db"), recursive=True))
    for path in files:
        rel = os.path.relpath(path, REFERENCE)
        con = sqlite3.connect(f"file:{path}?mode=ro", uri=True)
        have = {r[0] for r in con.execute("SELECT name FROM sqlite_master WHERE type='table'")}
        for table in TABLES:
            if table not in have:
                continue
            cols = [r[1] for r in con.execute(f"PRAGMA table_info({table})")]
            for row in con.execute(f"SELECT * FROM {table} WHERE rank = 0"):
                rec = dict(zip(cols, row))
                key = rec.pop("key")
                rec.pop("rank")
                for long, short in SHORT:
                    key = key.replace(long, short)
                entry = tables[table].setdefault(key, {"files": [], "rank0": rec})
                entry["files"].append(rel)
        con.close()
    doc = {"source": "benchmark/**/tuner_cache.db of apuaaChen/EVT_AE (keys abbreviated: h = cutlass::half_t, "
                     "R / C = cutlass::layout::RowMajor / ColumnMajor)",
           "epilogue_counts": ["aux_load", "row_broadcast", "column_broadcast", "aux_store", "row_reduction",
                               "column_reduction", "row_store"],
           "files": [os.path.relpath(p, REFERENCE) for p in files],
           "tables": {t: dict(sorted(v.items())) for t, v in tables.items()}}
    with open(OUT, "w") as f:      # one key per line
        tabs = doc.pop("tables")
        head = json.dumps(doc, indent=1)
        f.write(head[:head.rindex("}")].rstrip() + ',\n "tables": {\n')
        for ti, (t, rows) in enumerate(tabs.items()):
            f.write(f'  {json.dumps(t)}: {{\n')
            f.write(",\n".join(f"   {json.dumps(k)}: {json.dumps(v)}" for k, v in rows.items()))
            f.write("\n  }" + ("," if ti + 1 < len(tabs) else "") + "\n")
        f.write(" }\n}\n")
    print({t: len(v) for t, v in tables.items()})


if __name__ == "__main__":
    main()
