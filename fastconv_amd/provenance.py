"""Which kernel sources a measurement was taken with.

Every text summary under profiles/ carries one line

    provenance: commit <12 hex digits> csrc_sha256 <16 hex digits> [sources_sha256 <16 hex digits> <file> ...]

written by stamp(): the commit of the tree, a digest of all kernel sources (fastconv_amd/csrc/*.hip, *.h) and,
optionally, a digest of the few sources the numbers in that file depend on.  bench.py uses the last form to drop
measured HBM traffic once the kernels it was measured on have changed (roofline.traffic is then null, not stale).
"""
import glob
import hashlib
import os
import re
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
_LINE = re.compile(r"^provenance: commit ([0-9a-f]{12}) csrc_sha256 ([0-9a-f]{16})(?: sources_sha256 ([0-9a-f]{16})((?: \S+)+))?\s*$")


def digest(names=None, read=None):
    """sha256 (first 16 hex digits) over name and contents of the given files of csrc/, all *.hip and *.h when
    names is None.  `read(name) -> bytes` replaces reading from the working tree (used to digest an older commit)."""
    if names is None:
        names = sorted(os.path.basename(p) for p in glob.glob(os.path.join(CSRC, "*.hip")) + glob.glob(os.path.join(CSRC, "*.h")))
    h = hashlib.sha256()
    for n in sorted(names):
        data = read(n) if read else open(os.path.join(CSRC, n), "rb").read()
        h.update(n.encode() + b"\0" + data)
    return h.hexdigest()[:16]


def stamp(sources=None):
    """The provenance line for a summary written now from this working tree."""
    try:
        commit = subprocess.check_output(["git", "-C", _HERE, "rev-parse", "HEAD"], text=True, stderr=subprocess.DEVNULL).strip()[:12]
    except (OSError, subprocess.CalledProcessError):
        commit = "0" * 12
    line = "provenance: commit %s csrc_sha256 %s" % (commit, digest())
    if sources:
        line += " sources_sha256 %s %s" % (digest(sources), " ".join(sorted(sources)))
    return line


def parse(path):
    """(commit, csrc digest, sources digest or None, source names) of the provenance line of a summary, or None."""
    for line in open(path):
        m = _LINE.match(line)
        if m:
            return m.group(1), m.group(2), m.group(3), (m.group(4) or "").split()
    return None


def sources_current(path):
    """True when the summary names the sources it depends on and they are unchanged in this tree."""
    p = parse(path)
    if not p or not p[2]:
        return False
    try:
        return digest(p[3]) == p[2]
    except OSError:
        return False
