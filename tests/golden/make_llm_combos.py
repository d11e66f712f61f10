"""Writes llm_matmul_combos.json: the distinct attribute combinations of the quantized entries of the reference's LLM
matmul list (tests/benchdnn/inputs/matmul/option_set_fwks_llm_gpu), shapes dropped. Group sizes that equal the
entry's K are written as "K". Run where the reference tree is present:  python tests/golden/make_llm_combos.py"""
import collections
import json
import os
import re

LIST = "/root/reference/tests/benchdnn/inputs/matmul/option_set_fwks_llm_gpu"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "llm_matmul_combos.json")


def main():
    combos = collections.OrderedDict()
    for line in open(LIST):
        if not line.startswith("--reset"):
            continue
        o = dict(re.findall(r"--([a-z_-]+)=(\S*)", line))
        if o["dt"] == "f16:f16:f16":
            continue
        m = re.search(r"\s(\d+(?:x\d+)*):(\d+(?:x\d+)*)(?:_n|\s|$)", line)
        K = m.group(1).split("x")[-1]
        whole = lambda spec: re.sub(r"1x%s\b" % K, "1xK", spec)
        key = (o["dt"], o["stag"], o["wtag"], o["dtag"], whole(o.get("attr-scales", "")),
               whole(o.get("attr-zero-points", "")), o.get("attr-post-ops", ""), o.get("bia-dt", ""), o.get("bia_mask", ""),
               o.get("attr-fpmath", ""))
        combos[key] = combos.get(key, 0) + 1
    rows = [dict(dt=k[0], stag=k[1], wtag=k[2], dtag=k[3], scales=k[4], zero_points=k[5], post_ops=k[6], bia_dt=k[7],
                 bia_mask=k[8], fpmath=k[9], entries=n) for k, n in combos.items()]
    with open(OUT, "w") as f:
        f.write("[\n" + ",\n".join(json.dumps(r) for r in rows) + "\n]\n")
    print(len(rows), "combinations ->", OUT)


if __name__ == "__main__":
    main()
