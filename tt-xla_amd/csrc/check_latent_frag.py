#!/usr/bin/env python3
"""Build check for the kernels whose accumulators live in accumulation registers that no variable
stands for (gen_latent_frag.py, hidden_accumulators): in the compiled assembly of decode_wide.hip,
every kernel that holds a marked block may name an accumulation register only inside the marked
blocks, and may not spill (a spill could go through accumulation registers)."""
import re
import sys

BEGIN, END = "latent-frag accumulators begin", "latent-frag accumulators end"
AGPR = re.compile(r"\ba(\d+|\[\d+:\d+\])")


def main():
    text = open(sys.argv[1]).read().split("\n")
    kernel, inside, marked, bad = None, False, set(), []
    for line in text:
        m = re.match(r"^(_Z\w+):", line)
        if m:
            kernel, inside = m.group(1), False
            continue
        if kernel is None:
            continue
        if BEGIN in line:
            inside = True
            marked.add(kernel)
            continue
        if END in line:
            inside = False
            continue
        if "s_endpgm" in line:
            kernel = None if not line.strip().startswith("s_endpgm") else kernel
        code = line.split(";")[0]
        if not inside and code.strip() and not code.strip().startswith(".") and AGPR.search(code.split(None, 1)[1] if len(code.split(None, 1)) > 1 else ""):
            bad.append((kernel, line.strip()))
    bad = [(k, l) for k, l in bad if k in marked]
    for k in marked:
        m = re.search(re.escape(k) + r".*?\.amdhsa_private_segment_fixed_size (\d+)", "\n".join(text), re.S)
        if m and int(m.group(1)) != 0:
            bad.append((k, f"scratch: {m.group(1)} bytes per lane"))
    if not marked:
        print("check_latent_frag: no marked block found", file=sys.stderr)
        return 1
    for k, l in bad:
        print(f"check_latent_frag: {k}: {l}", file=sys.stderr)
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main())
