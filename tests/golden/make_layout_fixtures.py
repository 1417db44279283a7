#!/usr/bin/env python3
"""Extracts small layout fixtures from the reference's own tensor dumps (run in the build container only).

Reads  /root/reference/Leaf_Data_0.json and Node_Data_0.json  (llama.cpp dumps of LLaMA-3.1-8B-Q8_0: per tensor
the dims, ggml type, byte size and the FIRST 128 BYTES of data) and writes  q8_0_layout_fixtures.json  next to
this file:
  * for every Q8_0 tensor (ggml type 8): name, dims, byte_size            -> pins the byte-size formula
  * for a few of them the first 128 bytes (3 whole blocks + 26 bytes)     -> pins where d and qs sit in a block
  * the first 128 bytes (32 floats) of the `inp_embd` node, the dequantized embedding row of the first prompt token
                                                                          -> pins y = f32(d) * q
These are data the reference ships, not code.  Nothing here executes anything from the reference.
"""
import json
import os

REF = "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))
WITH_DATA = {"blk.0.attn_q.weight", "blk.0.attn_k.weight", "blk.0.ffn_down.weight", "blk.0.ffn_gate.weight", "token_embd.weight", "blk.31.attn_output.weight", "output.weight"}


def main() -> None:
    leaf = json.load(open(os.path.join(REF, "Leaf_Data_0.json")))
    node = json.load(open(os.path.join(REF, "Node_Data_0.json")))
    out = {"source": "reference Leaf_Data_0.json / Node_Data_0.json", "q8_0_tensors": [], "inp_embd": None}
    for e in leaf:
        if e["type"] != 8:
            continue
        item = {"name": e["name"], "dims": e["dims"], "byte_size": e["byte_size"]}
        if e["name"] in WITH_DATA:
            item["first_bytes"] = e["data"]
        out["q8_0_tensors"].append(item)
    for e in node:
        if e["name"] == "inp_embd":
            out["inp_embd"] = {"dims": e["dims"], "type": e["type"], "byte_size": e["byte_size"], "first_bytes": e["data"]}
            break
    with open(os.path.join(HERE, "q8_0_layout_fixtures.json"), "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print(len(out["q8_0_tensors"]), "q8_0 tensors;", sum("first_bytes" in t for t in out["q8_0_tensors"]), "with data")


if __name__ == "__main__":
    main()
