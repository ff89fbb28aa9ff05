"""Trim the reference's recorded search result into graph specs (data only).

Source (read as JSON data, nothing is imported or executed):
  <reference>/demo/checkpoint_group_query_attn_spec_decode.json
It holds the computation graph for GQA Q[2,256,64] K[2,64,4096] V[2,4096,64]
and the 69 candidate mugraphs the reference's own verify() accepted as
fingerprint-equal to it.  This script keeps, per graph, only what is needed to
rebuild it through a host API: op kinds, producer references (resolved from
tensor guids), dims/layouts of inputs, and each customized op's plan.  The
older schema has no `reduction_dimx`; the reference default 64 applies
(include/mirage/threadblock/graph.h:40).

It also keeps an excerpt of the file in its ORIGINAL schema: the whole checkpoint object
(include/mirage/search/search.h:46-68: best_graph, best_profile_result, config, callstack,
the three counters, the computation graph) with every ninth generated graph, verbatim JSON
objects: the data the JSON wire format and the checkpoint loader of the host API are
tested against.

Usage: python tests/golden/extract_gqa_checkpoint.py [reference_root]
Writes tests/golden/gqa_spec_decode_69.json and
tests/golden/gqa_spec_decode_checkpoint_excerpt.json
"""
import json
import os
import sys

KN = {
    "kn_input_op": "input", "kn_matmul_op": "matmul", "kn_exp_op": "exp",
    "kn_add_op": "add", "kn_mul_op": "mul", "kn_div_op": "div",
    "kn_customized_op": "customized",
}


def convert(ops):
    producer = {}
    out = []
    for i, op in enumerate(ops):
        t = op["op_type"]
        rec = {}
        if t.startswith("kn_reduction_"):
            rec["op"] = "reduction"
            rec["dim"] = int(t[len("kn_reduction_")])
            rec["size"] = op["output_tensors"][0]["dim"][rec["dim"]]
        else:
            rec["op"] = KN[t]
        if rec["op"] == "input":
            ot = op["output_tensors"][0]
            rec["dims"] = ot["dim"][: ot["num_dims"]]
            rec["layout"] = ot["layout"]
        else:
            rec["in"] = [list(producer[x["guid"]]) for x in op["input_tensors"]]
        if rec["op"] == "customized":
            p = op["plan"]
            xyz = lambda d: [d["x"], d["y"], d["z"]]
            rec["plan"] = {
                "grid_dim": xyz(p["grid_dim"]), "block_dim": xyz(p["block_dim"]),
                "forloop_range": p["forloop_range"],
                "reduction_dimx": p.get("reduction_dimx", 64),
                "input_map": [xyz(m) for m in p["input_map"]],
                "forloop_dim": p["forloop_dim"],
                "output_map": xyz(p["output_map"]),
                "input_smem_layouts": p["input_smem_layouts"],
                "ops": p["ops"],
            }
            rec["smem_offset"] = op["bgraph"]["smem_offset"]
        rec["out_dims"] = [x["dim"][: x["num_dims"]] for x in op["output_tensors"]]
        for j, x in enumerate(op["output_tensors"]):
            producer[x["guid"]] = (i, j)
        out.append(rec)
    return out


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    src = os.path.join(root, "demo", "checkpoint_group_query_attn_spec_decode.json")
    j = json.load(open(src))
    doc = {
        "source": "demo/checkpoint_group_query_attn_spec_decode.json",
        "num_total_kernel_graphs": j["num_total_kernel_graphs"],
        "num_total_random_tests": j["num_total_random_tests"],
        "num_valid_kernel_graphs": j["num_valid_kernel_graphs"],
        "computation_graph": convert(j["computation_graph"]),
        "generated_graphs": [convert(g) for g in j["generated_graphs"]],
    }
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gqa_spec_decode_69.json")
    with open(dst, "w") as f:
        json.dump(doc, f, separators=(",", ":"))
    picks = list(range(0, len(j["generated_graphs"]), 9))
    excerpt = {k: v for k, v in j.items() if k != "generated_graphs"}
    excerpt.update({
        "source": "demo/checkpoint_group_query_attn_spec_decode.json",
        "indices": picks,
        "generated_graphs": [j["generated_graphs"][i] for i in picks],
    })
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)),
                       "gqa_spec_decode_checkpoint_excerpt.json")
    with open(dst, "w") as f:
        json.dump(excerpt, f, separators=(",", ":"), sort_keys=True)
    print(dst, os.path.getsize(dst), "bytes,", len(doc["generated_graphs"]), "graphs")


if __name__ == "__main__":
    main()
