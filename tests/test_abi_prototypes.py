"""Header prototypes against the reference's own definitions (CPU; skipped where the reference tree is absent).

Every function the header shares with adamah-MAIN/adamah/adamah.c must take the same argument types in the same
order and return the same type, except where the reference's Python binding reads the return value as a 64-bit
ticket although the C function says int -- there the header follows the binding (its `restype` lines are read
from adamah/__init__.py)."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "adamah_hip.h")
REF_C = "/root/reference/adamah-MAIN/adamah/adamah.c"
REF_PY = "/root/reference/adamah-MAIN/adamah/__init__.py"

pytestmark = pytest.mark.skipif(not (os.path.exists(REF_C) and os.path.exists(REF_PY)), reason="reference tree not present")


def _strip_comments(src):
    src = re.sub(r"/\*.*?\*/", " ", src, flags=re.S)
    return re.sub(r"//[^\n]*", " ", src)


def _norm_type(arg):
    """'const uint32_t *locs' -> 'const uint32_t*'; the parameter name goes, spelling of the type stays."""
    arg = " ".join(arg.replace("*", " * ").split())
    if arg in ("void", ""):
        return None
    toks = arg.split(" ")
    if toks[-1] != "*" and len(toks) > 1:
        toks = toks[:-1]                       # drop the name
    return "".join(t if t == "*" else (" " + t) for t in toks).strip().replace(" *", "*")


def _prototypes(src, definitions):
    """name -> (return type, [argument types]).  definitions=True: 'type name(args) {' at the start of a line."""
    out = {}
    tail = r"\{" if definitions else r";"
    for m in re.finditer(r"(?m)^(?:extern\s+)?([A-Za-z_][\w \t\*]*?)\s*\b((?:adamah_|map_|batch_)\w+)\s*\(([^()]*)\)\s*" + tail, src):
        ret, name, args = m.group(1), m.group(2), m.group(3)
        if "static" in ret.split() or "return" in ret.split():
            continue
        types = [t for t in (_norm_type(a) for a in args.split(",")) if t]
        out[name] = (" ".join(ret.replace("*", " * ").split()).replace(" *", "*"), types)
    return out


def test_shared_functions_have_the_reference_signatures():
    ours = _prototypes(_strip_comments(open(HEADER).read()), definitions=False)
    ref = _prototypes(_strip_comments(open(REF_C).read()), definitions=True)
    shared = sorted(set(ours) & set(ref))
    assert len(shared) >= 90, len(shared)
    binding = open(REF_PY).read()
    ticket64 = set(re.findall(r"self\._lib\.(\w+)\.restype\s*=\s*ctypes\.c_uint64", binding))
    wrong = []
    for name in shared:
        (r_o, a_o), (r_r, a_r) = ours[name], ref[name]
        if a_o != a_r:
            wrong.append((name, "arguments", a_o, a_r))
        if r_o != r_r and not (r_o == "uint64_t" and r_r == "int" and name in ticket64):
            wrong.append((name, "return", r_o, r_r))
    assert not wrong, wrong


def test_return_types_that_follow_the_binding_are_the_four_ticket_calls():
    ours = _prototypes(_strip_comments(open(HEADER).read()), definitions=False)
    ref = _prototypes(_strip_comments(open(REF_C).read()), definitions=True)
    differ = sorted(n for n in set(ours) & set(ref) if ours[n][0] != ref[n][0])
    assert differ == ["map_gather", "map_scatter", "map_scatter_contiguous", "map_scatter_q4_packed_contiguous"], differ
