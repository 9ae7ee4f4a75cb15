#!/usr/bin/env python3
"""Cut the data fixtures this repository's tests use out of the reference's test resources.

Run in the build container only (the reference tree is not present on the GPU box):

    python tests/golden/make_fixtures.py [/root/reference]

Outputs (committed; pure data, no reference code):
  tests/golden/fixture.gguf       byte copy of jitnn-gguf/src/test/resources/gguf/fixture.gguf
  tests/golden/golden_cases.bin   the arrays of the selected golden cases, concatenated
  tests/golden/golden_cases.txt   manifest in the reference's own format
                                  (jitnn-core/src/test/java/ai/beestream/jitnn/Golden.java:79-123):
                                    case <name> <op> <attrs...>
                                    <case> <array> <f32|i32> <byte offset> <dims...>
                                  with offsets rebased to golden_cases.bin.

Only inputs (in*) and expected outputs (out) are kept: gradients and the autograd helper array
"w" are not part of the quantised linear path.
"""
import re
import shutil
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent

# gguf_* pin the dequantisers and the GEMV; the rest pin the decode-step glue and seeded inputs.
SELECT = re.compile(
    r"^(gguf_(linear|dequant)_.*|rms_norm(_3d|_long|_rows)?|rope_heads|rope_heads_interleaved|"
    r"rope_half|rope_offset|rope_long|sdpa_bthd_causal|sdpa_head128|sdpa_causal|sdpa|silu|silu_tails|"
    r"swiglu|embedding|matmul_t01_.*|init_uniform)$"
)
KEEP_ARRAY = re.compile(r"^(in\d+|out)$")


def main() -> None:
    ref = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    shutil.copyfile(ref / "jitnn-gguf/src/test/resources/gguf/fixture.gguf", HERE / "fixture.gguf")

    gold = ref / "jitnn-core/src/test/resources/golden"
    data = (gold / "data.bin").read_bytes()
    out_bin = bytearray()
    out_txt = ["# cut from the reference's golden/manifest.txt + data.bin by make_fixtures.py"]
    wanted = set()
    for line in (gold / "manifest.txt").read_text().splitlines():
        t = line.split()
        if len(t) < 2 or t[0].startswith("#"):
            continue
        if t[0] == "case":
            if SELECT.match(t[1]):
                wanted.add(t[1])
                out_txt.append(line.strip())
            continue
        if t[0] not in wanted or not KEEP_ARRAY.match(t[1]):
            continue
        dims = [int(d) for d in t[4:]]
        n = 1
        for d in dims:
            n *= d
        off = int(t[3])
        new_off = len(out_bin)
        out_bin += data[off:off + 4 * n]
        out_txt.append(" ".join([t[0], t[1], t[2], str(new_off)] + [str(d) for d in dims]))
    (HERE / "golden_cases.bin").write_bytes(bytes(out_bin))
    (HERE / "golden_cases.txt").write_text("\n".join(out_txt) + "\n")
    print(f"{len(wanted)} cases, {len(out_bin)} bytes")


if __name__ == "__main__":
    main()
