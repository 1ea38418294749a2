#!/usr/bin/env python3
"""Build step: read hipcc's -Rpass-analysis=kernel-resource-usage remarks for one translation unit and fail when a
kernel spills too much to scratch (private) memory.

    python3 check_resources.py build/<unit>.log [LIMIT_BYTES [NO_SCRATCH_REGEX]]

Two reasons.  A kernel whose loops were unrolled into hundreds of live values can ask for tens of KB of scratch per
lane, and a launch of such a kernel fails at run time for lack of scratch memory: no kernel may use more than
LIMIT_BYTES (default 256) per lane.  And a kernel that consumes inline-assembly loads after a hand-counted
s_waitcnt relies on the loaded registers not being spilled in between: kernels whose name matches
NO_SCRATCH_REGEX may use none at all.
Writes a one-line-per-kernel summary next to the log (<unit>.resources.txt).
"""
import re
import sys


def main():
    path = sys.argv[1]
    limit = int(sys.argv[2]) if len(sys.argv) > 2 else 256
    none = re.compile(sys.argv[3]) if len(sys.argv) > 3 else None
    text = open(path, errors="replace").read()
    rows, cur = [], None
    for line in text.splitlines():
        m = re.search(r"remark: .*Function Name: (\S+)", line)
        if m:
            cur = {"name": m.group(1)}
            rows.append(cur)
            continue
        if cur is None:
            continue
        for key, pat in (("vgprs", r"remark:.*\bVGPRs: (\d+)"), ("agprs", r"remark:.*\bAGPRs: (\d+)"),
                         ("sgprs", r"remark:.*\bSGPRs: (\d+)"), ("scratch", r"remark:.*ScratchSize \[bytes/lane\]: (\d+)"),
                         ("occupancy", r"remark:.*Occupancy \[waves/SIMD\]: (\d+)"),
                         ("lds", r"remark:.*LDS Size \[bytes/block\]: (\d+)")):
            m = re.search(pat, line)
            if m:
                cur[key] = int(m.group(1))
    out = path.rsplit(".", 1)[0] + ".resources.txt"
    bad = []
    with open(out, "w") as f:
        for r in rows:
            f.write("{name} vgprs={vgprs} agprs={agprs} sgprs={sgprs} scratch={scratch} occupancy={occupancy} lds={lds}\n"
                    .format(**{k: r.get(k, "?") for k in ("name", "vgprs", "agprs", "sgprs", "scratch", "occupancy", "lds")}))
            if r.get("scratch", 0) > (0 if none and none.search(r["name"]) else limit):
                bad.append(r)
    for r in bad:
        sys.stderr.write(f"check_resources: {r['name']} uses {r['scratch']} bytes of scratch per lane\n")
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main())
