"""Extracts, from the expected `qwen info` output the reference's own CLI test holds
(crates/qwen-cli/tests/fixtures/run-front-info-cli-v1.json, checked by tests/run_front_info.rs), the facts a GGUF
reader must reproduce for the fixture files next to it (crates/qwen-cli/tests/fixtures/run-front-models/*.gguf, copied
to tests/golden/gguf/): tensor count, where the tensor data starts, the tensors of block 0 in file order and the
architecture's metadata values.  Reads data files only; writes tests/golden/gguf/expected_info.json."""
import json
import os
import re
import sys

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    base = json.load(open(os.path.join(REF, "crates/qwen-cli/tests/fixtures/run-front-info-cli-v1.json")))
    out = {}
    for arch in ("qwen35", "qwen35moe"):
        text = base[arch]["text_utf8"]
        m = re.search(r"arch=(\S+) (\d+) tensors, (\d+) shard\(s\), .* tensor-data starts at (\d+)", text)
        lines = text.splitlines()
        i = next(k for k, l in enumerate(lines) if l.startswith("blk.0 tensors"))
        n = int(re.search(r"\((\d+)\)", lines[i]).group(1))
        blk0 = [l.strip() for l in lines[i + 1:i + 1 + n]]
        j = next(k for k, l in enumerate(lines) if l.startswith("metadata ("))
        meta = {}
        for l in lines[j + 1:]:
            mm = re.match(r"  (\S+) = (\d+)$", l)
            if not mm:
                break
            meta[mm.group(1)] = int(mm.group(2))
        out[arch] = {"architecture": m.group(1), "tensors": int(m.group(2)), "data_start": int(m.group(4)),
                     "blk0_tensors": blk0, "metadata": meta}
    with open(os.path.join(HERE, "gguf", "expected_info.json"), "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
        f.write("\n")


if __name__ == "__main__":
    main()
