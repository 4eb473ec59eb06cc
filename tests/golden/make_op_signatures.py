"""Writes tests/golden/op_signatures.json: for every operator the reference's extension exports (`m.def` in
fast_2d_gs/_C/src/**/*.cu), the positional parameters of its host function -- name, whether it is an optional tensor
(`torch::optional<...>`), and whether the binding gives it a default (`py::arg(...) = value`).

Run in the build container (reads the reference's sources as text, imports nothing from them):
    python tests/golden/make_op_signatures.py /root/reference
The JSON holds data only (names and flags); tests/test_boundary.py compares it with inspect.signature of the operators
in fast_sp_gs_amd/_C/_ops.py.
"""
import json
import re
import sys
from pathlib import Path


def split_top(text: str):
    out, depth, cur = [], 0, ''
    for ch in text:
        if ch in '<([{':
            depth += 1
        elif ch in '>)]}':
            depth -= 1
        if ch == ',' and depth == 0:
            out.append(cur.strip())
            cur = ''
        else:
            cur += ch
    if cur.strip():
        out.append(cur.strip())
    return out


def strip_comments(src: str) -> str:
    src = re.sub(r'/\*.*?\*/', '', src, flags=re.S)
    return re.sub(r'//[^\n]*', '', src)


def main(ref_root: str):
    root = Path(ref_root) / 'fast_2d_gs' / '_C' / 'src'
    table = {}
    for path in sorted(root.rglob('*.cu')):
        src = strip_comments(path.read_text(errors='replace'))
        for m in re.finditer(r'm\.def\(\s*"(\w+)"\s*,\s*&?\s*(\w+)([^;]*)\)\s*;', src, flags=re.S):
            py_name, c_name, rest = m.group(1), m.group(2), m.group(3)
            defaults = set(re.findall(r'py::arg\("(\w+)"\)\s*=', rest))
            # the host function's definition: `<return type> c_name(<params>) {`
            d = re.search(r'[\w:<>,\s\*&]+?\b' + re.escape(c_name) + r'\s*\(', src)
            defs = [x for x in re.finditer(r'\b' + re.escape(c_name) + r'\s*\(', src)]
            params = None
            for x in defs:
                i, depth = x.end(), 1
                while i < len(src) and depth:
                    depth += src[i] == '('
                    depth -= src[i] == ')'
                    i += 1
                after = src[i:i + 40].lstrip()
                if after.startswith('{'):  # a definition, not a call or a declaration
                    params = split_top(src[x.end():i - 1])
                    break
            if params is None:
                continue
            entry = []
            for p_ in params:
                p_ = re.sub(r'\s+', ' ', p_)
                if p_ in ('', 'void'):
                    continue
                name = re.findall(r'(\w+)\s*(?:=.*)?$', p_)[0]
                entry.append({'name': name, 'optional': 'optional<' in p_, 'default': name in defaults})
            table[py_name] = {'file': str(path.relative_to(Path(ref_root))), 'params': entry}
    out = Path(__file__).with_name('op_signatures.json')
    out.write_text(json.dumps(table, indent=1, sort_keys=True) + '\n')
    print(f'{len(table)} operators -> {out}')


if __name__ == '__main__':
    main(sys.argv[1] if len(sys.argv) > 1 else '/root/reference')
