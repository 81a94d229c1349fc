"""Writes tests/golden/rules_pairs.json: the ordered hand pairs asserted by the reference's
``tests/test_rules.py`` (``assert_all_compares(a, b, expected)`` call sites), restated as
data.  The reference file is parsed as text with ``ast``; nothing from it is imported or
run.  Calls wrapped in ``try`` (input-robustness tests that accept any outcome) are skipped.

Run once, here only:  python tests/golden/extract_rules_pairs.py
"""
import ast
import json
import os

SRC = "/root/reference/tests/test_rules.py"
HERE = os.path.dirname(os.path.abspath(__file__))


def C(r, s):
    return s * 13 + r


def ev(node, env):
    return eval(compile(ast.Expression(node), "<expr>", "eval"), {"C": C}, env)


def main():
    tree = ast.parse(open(SRC).read())
    pairs = []
    for fn in tree.body:
        if not isinstance(fn, ast.FunctionDef) or not fn.name.startswith("test_"):
            continue
        in_try = set()
        for node in ast.walk(fn):
            if isinstance(node, ast.Try):
                in_try.update(id(x) for x in ast.walk(node))
        env = {}
        for st in ast.walk(fn):
            if isinstance(st, ast.Assign) and len(st.targets) == 1 and isinstance(st.targets[0], ast.Name):
                try:
                    env[st.targets[0].id] = ev(st.value, env)
                except Exception:
                    pass
        for st in ast.walk(fn):
            if isinstance(st, ast.Call) and getattr(st.func, "id", "") == "assert_all_compares" and id(st) not in in_try:
                a, b, e = (ev(x, env) for x in st.args)
                pairs.append({"test": fn.name, "a": a, "b": b, "expected": e})
    out = {"source": "tests/test_rules.py of the reference (assert_all_compares call sites)", "pairs": pairs}
    with open(os.path.join(HERE, "rules_pairs.json"), "w") as f:
        json.dump(out, f, indent=0)
    print(len(pairs), "pairs")


if __name__ == "__main__":
    main()
