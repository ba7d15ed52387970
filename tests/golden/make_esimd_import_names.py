#!/usr/bin/env python3
"""Writes tests/golden/esimd_import_names.json: every name the reference's patched callers read
from the kernel packages `custom_esimd_kernels_vllm` / `custom_esimd_kernels_sglang`, read as
TEXT from the two patch files.  Nothing from the reference is imported or run.

    python tests/golden/make_esimd_import_names.py [/root/reference]

Two kinds of site are recorded, each with the patch line it stands on:
  * attribute reads on the import-safe handle of the patched vLLM's esimd_utils.py
    (`_esimd.<name>`, `_esimd.<module>.<name>`; vllm/patches/vllm_for_multi_arc.patch:2972-3252) --
    "guarded" when the read is a `getattr(_esimd, "<name>", None)` / `hasattr(_esimd, "<name>")`;
  * `from <package>[.<module>] import <names>` and `import <package>.<module>` statements anywhere
    in the patches -- "guarded" when an enclosing block is a `try:`.
An unguarded name that the package lacks breaks the caller's import; a guarded one makes the
caller fall back.  tests/test_capi_cpu.py holds the package to that.

Also recorded, as plain name lists:
  * "sglang_package_exports": the `_EXPORTS` list of the reference's SGLang package
    (sglang/custom-esimd-kernels/python/custom_esimd_kernels_sglang/__init__.py), the module-level
    names it re-exports from its ops.py when their extension is built;
  * "imp_kernels_names": the names the patched SGLang takes through its `_imp_kernels((...))` helper
    (sglang package first, vLLM package second, else None; sglang_for_multi_arc.patch:2077-2140).
"""
import json
import os
import re
import sys

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
PATCHES = {
    "vllm": "vllm/patches/vllm_for_multi_arc.patch",
    "sglang": "sglang/patches/sglang_for_multi_arc.patch",
}
PKGS = ("custom_esimd_kernels_vllm", "custom_esimd_kernels_sglang")
ATTR = re.compile(r"(?<![\w.])_esimd\.([A-Za-z_]\w*)(?:\.([A-Za-z_]\w*))?")
SOFT = re.compile(r"(?<![\w.])_esimd\s*,\s*\"([A-Za-z_]\w*)\"")   # getattr / hasattr, possibly wrapped
FROM = re.compile(r"^from\s+(custom_esimd_kernels_(?:vllm|sglang))((?:\.\w+)*)\s+import\s+(.*)$")
IMPORT = re.compile(r"^import\s+(custom_esimd_kernels_(?:vllm|sglang))\.(\w+)")


def added_lines(path):
    """(patch line number, text without the leading '+') of every added line, with the file
    of the diff it belongs to."""
    cur = None
    for no, line in enumerate(open(path, errors="replace"), 1):
        if line.startswith("diff --git"):
            cur = line.split(" b/", 1)[1].strip()
        elif line.startswith("+") and not line.startswith("+++"):
            yield no, cur, line[1:].rstrip("\n")
        elif line.startswith(" "):
            yield no, cur, line[1:].rstrip("\n")


def indent(s):
    return len(s) - len(s.lstrip(" "))


def in_try(lines, i):
    """True when a block enclosing lines[i] opens with `try:`."""
    ind = indent(lines[i][2])
    for j in range(i - 1, -1, -1):
        if lines[j][1] != lines[i][1]:
            break
        t = lines[j][2]
        if not t.strip() or t.lstrip().startswith("#"):
            continue
        k = indent(t)
        if k < ind:
            if t.strip() == "try:":
                return True
            ind = k
            if k == 0:
                break
    return False


def import_names(lines, i, tail):
    """Names of a `from ... import a, b as c` / parenthesised multi-line import."""
    text = tail
    if "(" in tail and ")" not in tail:
        j = i + 1
        while j < len(lines) and ")" not in lines[j][2]:
            text += " " + lines[j][2]
            j += 1
        if j < len(lines):
            text += " " + lines[j][2]
    text = re.sub(r"#.*", "", text.replace("(", " ").replace(")", " "))
    out = []
    for part in text.split(","):
        part = part.strip()
        if part:
            out.append(part.split(" as ")[0].strip())
    return out


def main():
    result = {"esimd_utils_reads": [], "imports": []}
    for which, rel in PATCHES.items():
        lines = list(added_lines(os.path.join(REF, rel)))
        for i, (no, fname, text) in enumerate(lines):
            body = text.strip()
            if fname and fname.endswith("layers/esimd_utils.py") and not body.startswith("#"):
                for m in SOFT.finditer(text):
                    result["esimd_utils_reads"].append(
                        {"line": no, "module": None, "name": m.group(1), "guarded": True})
                for m in ATTR.finditer(text):
                    mod, name = (m.group(1), m.group(2)) if m.group(2) else (None, m.group(1))
                    result["esimd_utils_reads"].append(
                        {"line": no, "module": mod, "name": name, "guarded": False})
            m = FROM.match(body)
            if m:
                result["imports"].append({
                    "patch": which, "line": no, "package": m.group(1), "module": m.group(2).lstrip(".") or None,
                    "names": import_names(lines, i, m.group(3)), "guarded": in_try(lines, i)})
                continue
            m = IMPORT.match(body)
            if m:
                result["imports"].append({
                    "patch": which, "line": no, "package": m.group(1), "module": m.group(2),
                    "names": [], "guarded": in_try(lines, i)})
    init = open(os.path.join(REF, "sglang/custom-esimd-kernels/python/custom_esimd_kernels_sglang/__init__.py")).read()
    block = init[init.index("_EXPORTS = ["):init.index("]", init.index("_EXPORTS = ["))]
    result["sglang_package_exports"] = re.findall(r'"([A-Za-z_]\w*)"', block)
    imp = set()
    for _, _, text in added_lines(os.path.join(REF, PATCHES["sglang"])):
        if "_imp_kernels(" in text and "def _imp_kernels" not in text:
            imp.update(re.findall(r'"([A-Za-z_]\w*)"', text))
    # multi-line calls: the tuple continues on the next line
    lines = [t for _, _, t in added_lines(os.path.join(REF, PATCHES["sglang"]))]
    for i, t in enumerate(lines):
        if t.rstrip().endswith("_imp_kernels("):
            imp.update(re.findall(r'"([A-Za-z_]\w*)"', lines[i + 1]))
    result["imp_kernels_names"] = sorted(imp)
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "esimd_import_names.json")
    with open(out, "w") as f:
        json.dump(result, f, indent=1, sort_keys=True)
        f.write("\n")
    print(f"{len(result['esimd_utils_reads'])} handle reads, {len(result['imports'])} import sites -> {out}")


if __name__ == "__main__":
    main()
