#!/usr/bin/env python3
"""Extracts the reference's ctest invocations of `single_conv_layer` and
`general_matrix_multiply` into JSON fixtures (data only: test names and
argument lists).

    python3 tests/golden/extract_ctest_matrix.py [/root/reference]

reads <reference>/tests/poplin/CMakeLists.txt, interprets the few CMake
commands that file uses around its tests (set, foreach / endforeach over
literal lists and RANGE, if / elseif / else / endif - every branch is taken,
a test's platform conditions do not matter here) and writes
tests/golden/<tool>_ctest_matrix.json for each of the two tools: one record
per add_multitarget_test / add_test whose COMMAND is that tool, with ${VAR}
references substituted.  Plan-constraint files the invocations name
(tests/poplin/json/*.json: data the reference holds) are copied next to the
fixture and the arguments rewritten to "@golden/<file>".  Runs only where the
reference tree is present; the GPU tests read the fixture, never the tree.
"""
import json
import os
import re
import shutil
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
TOOLS = ("single_conv_layer", "general_matrix_multiply")
REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
SRC = os.path.join(REF, "tests", "poplin", "CMakeLists.txt")


def tokenize(text):
    """CMake commands as (name, [arguments], line)."""
    text = re.sub(r"(?m)^\s*#.*$", "", text)
    out, i, n = [], 0, len(text)
    ident = re.compile(r"\s*([A-Za-z_][A-Za-z0-9_]*)\s*\(")
    while True:
        m = ident.match(text, i)
        if not m:
            rest = text[i:].strip()
            if rest:
                # skip stray text up to the next line
                j = text.find("\n", i)
                if j < 0:
                    break
                i = j + 1
                continue
            break
        line = text.count("\n", 0, m.start(1)) + 1
        i = m.end()
        args, cur, depth, quoted = [], "", 1, False
        while i < n and depth:
            c = text[i]
            if quoted:
                if c == "\\" and i + 1 < n:
                    cur += text[i + 1]
                    i += 2
                    continue
                if c == '"':
                    quoted = False
                    args.append(cur)
                    cur = ""
                    i += 1
                    continue
                cur += c
            elif c == '"' and not cur:
                quoted = True
            elif c == "#":
                j = text.find("\n", i)
                i = n if j < 0 else j
                continue
            elif c == "(":
                depth += 1
                cur += c
            elif c == ")":
                depth -= 1
                if depth:
                    cur += c
            elif c.isspace():
                if cur:
                    args.append(cur)
                    cur = ""
            elif c == "\\" and i + 1 < n:
                cur += text[i + 1]
                i += 1
            else:
                cur += c
            i += 1
        if cur:
            args.append(cur)
        out.append((m.group(1).lower(), args, line))
    return out


def substitute(s, env):
    for _ in range(8):
        t = re.sub(r"\$\{([A-Za-z0-9_]+)\}",
                   lambda m: env.get(m.group(1), m.group(0)), s)
        if t == s:
            break
        s = t
    return s


def run(cmds, env, tests):
    i = 0
    while i < len(cmds):
        name, args, line = cmds[i]
        if name == "foreach":
            depth, j = 1, i + 1
            while depth:
                if cmds[j][0] == "foreach":
                    depth += 1
                elif cmds[j][0] == "endforeach":
                    depth -= 1
                j += 1
            body = cmds[i + 1:j - 1]
            var = args[0]
            items = [substitute(a, env) for a in args[1:]]
            if items and items[0] == "RANGE":
                lo, hi = (0, int(items[1])) if len(items) == 2 else \
                    (int(items[1]), int(items[2]))
                items = [str(v) for v in range(lo, hi + 1)]
            else:
                flat = []
                for it in items:
                    flat += [x for x in it.split(";") if x != ""]
                items = flat
            for it in items:
                run(body, dict(env, **{var: it}), tests)
                # (set() inside a loop body is local to this interpretation)
            i = j
            continue
        if name == "set" and args:
            env[args[0]] = ";".join(substitute(a, env) for a in args[1:])
        elif name in ("add_multitarget_test", "add_test", "add_unit_test"):
            a = [substitute(x, env) for x in args]
            if "COMMAND" in a and "NAME" in a:
                k = a.index("COMMAND")
                if k + 1 < len(a) and a[k + 1] in TOOLS:
                    rest = a[k + 2:]
                    stops = {"VARIANTS", "LABELS", "ALLOW_SKIP", "TEST_IPUMODEL",
                             "PROPERTIES", "WORKING_DIRECTORY", "NAME"}
                    argv = []
                    for x in rest:
                        if x in stops:
                            break
                        argv.append(x)
                    tests.append({"name": a[a.index("NAME") + 1],
                                  "tool": a[k + 1], "line": line,
                                  "args": argv})
        i += 1


def main():
    with open(SRC) as f:
        cmds = tokenize(f.read())
    env = {"CMAKE_CURRENT_SOURCE_DIR": "@ref/tests/poplin",
           "CMAKE_SOURCE_DIR": "@ref"}
    tests = []
    run(cmds, env, tests)
    copied = set()
    for t in tests:
        for k, a in enumerate(t["args"]):
            m = re.search(r"@ref/tests/poplin/json/([A-Za-z0-9_.-]+\.json)", a)
            if m:
                name = m.group(1)
                if name not in copied:
                    shutil.copyfile(
                        os.path.join(REF, "tests", "poplin", "json", name),
                        os.path.join(HERE, name))
                    copied.add(name)
                t["args"][k] = a.replace(m.group(0), "@golden/" + name)
    names = {}
    for t in tests:  # (loops can repeat a name; ctest would refuse, we number)
        names[t["name"]] = names.get(t["name"], 0) + 1
        if names[t["name"]] > 1:
            t["name"] += f"#{names[t['name']]}"
    for tool in TOOLS:
        mine = [{k: v for k, v in t.items() if k != "tool"}
                for t in tests if t["tool"] == tool]
        out = os.path.join(HERE, tool + "_ctest_matrix.json")
        with open(out, "w") as f:
            json.dump({"source": "tests/poplin/CMakeLists.txt",
                       "tool": tool, "tests": mine}, f, indent=1)
            f.write("\n")
        print(f"{len(mine)} invocations -> {out}")
    print(f"constraint files copied: {sorted(copied)}")


if __name__ == "__main__":
    main()
