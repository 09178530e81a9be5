"""Writes tests/golden/worker_protocol.json from the data the reference's own
service tests hold (tests/server/test_expert_server.py): every scripted
worker's ready line together with the launch arguments of the worker client
that reads it, whether the client accepts it, the attribute values the test
asserts afterwards - and the literal command lines those tests expect on the
wire.  The test file is read as text and walked as a syntax tree; nothing of
the reference is imported or run.

    python tests/golden/make_worker_protocol_fixture.py [/root/reference]
"""
import ast
import json
import os
import sys

POSITIONAL = ("executable", "container", "max_context", "startup_timeout",
              "requested_capacity", "ram_cache_gib", "vram_cache_gib", "kv_cache_mib",
              "kv_page_tokens", "placement_profile", "profile_gpu_phases")
VERBS = ("BEGIN", "END", "DROP", "STEP", "NEXT", "CANCEL", "SAVE", "LOAD", "PRUNE",
         "\tSAMPLING")


def constant(node, names):
    """Literal value of an expression made of constants, containers, shifts,
    sums and products, the loop variables in `names`, and Path("x") -> "x"."""
    if isinstance(node, ast.Constant):
        return node.value
    if isinstance(node, ast.Name) and node.id in names:
        return names[node.id]
    if isinstance(node, (ast.Tuple, ast.List)):
        return [constant(item, names) for item in node.elts]
    if isinstance(node, ast.Dict):
        return {constant(key, names): constant(value, names)
                for key, value in zip(node.keys, node.values)}
    if isinstance(node, ast.BinOp):
        left, right = constant(node.left, names), constant(node.right, names)
        if isinstance(node.op, ast.LShift):
            return left << right
        if isinstance(node.op, ast.Mult):
            return left * right
        if isinstance(node.op, ast.Add):
            return left + right
    if isinstance(node, ast.Call) and getattr(node.func, "attr", "") == "Path":
        return constant(node.args[0], names)
    raise ValueError(ast.dump(node))


def is_raises(with_node):
    return any(isinstance(item.context_expr, ast.Call) and
               getattr(item.context_expr.func, "attr", "").startswith("assertRaises")
               for item in with_node.items)


def walk(body, names, ready, rejected, cases, function):
    """Statements in order, tracking the `ready` literal, loop variables and
    whether we are inside an assertRaises block."""
    for statement in body:
        if isinstance(statement, ast.Assign) and len(statement.targets) == 1:
            target = statement.targets[0]
            if isinstance(target, ast.Name) and target.id == "ready":
                try:
                    ready.clear()
                    ready.update(constant(statement.value, names))
                except ValueError:
                    ready.clear()
                continue
            if (isinstance(target, ast.Subscript) and
                    getattr(target.value, "id", "") == "ready" and ready):
                ready[constant(target.slice, names)] = constant(statement.value, names)
                continue
        if isinstance(statement, ast.For) and isinstance(statement.target, ast.Name):
            try:
                values = constant(statement.iter, names)
            except ValueError:
                continue
            for value in values:
                walk(statement.body, {**names, statement.target.id: value}, ready,
                     rejected, cases, function)
            continue
        if isinstance(statement, ast.With):
            walk(statement.body, names, ready, rejected or is_raises(statement), cases,
                 function)
            continue
        for node in ast.walk(statement):
            if (isinstance(node, ast.Call) and getattr(node.func, "id", "") == "CudaWorker"
                    and ready.get("type") == "ready"):
                launch = dict(zip(POSITIONAL, (constant(arg, names) for arg in node.args)))
                for keyword in node.keywords:
                    launch[keyword.arg] = constant(keyword.value, names)
                cases.append({"test": function, "ready": dict(ready), "launch": launch,
                              "accepted": not rejected, "attributes": {}})
            # assertEqual(worker.<attribute>, <literal>) after an accepted launch
            if (isinstance(node, ast.Call) and
                    getattr(node.func, "attr", "") in ("assertEqual", "assertTrue",
                                                       "assertFalse") and cases and
                    cases[-1]["test"] == function and node.args and
                    isinstance(node.args[0], ast.Attribute) and
                    getattr(node.args[0].value, "id", "") == "worker"):
                kind = node.func.attr
                try:
                    value = (constant(node.args[1], names) if kind == "assertEqual"
                             else kind == "assertTrue")
                except (ValueError, IndexError):
                    continue
                cases[-1]["attributes"][node.args[0].attr] = value


def main():
    reference = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    path = os.path.join(reference, "tests", "server", "test_expert_server.py")
    with open(path, encoding="utf-8") as source:
        tree = ast.parse(source.read())
    cases, lines = [], []
    for node in ast.walk(tree):
        if isinstance(node, ast.FunctionDef) and node.name.startswith("test_"):
            walk(node.body, {}, {}, False, cases, node.name)
            for inner in ast.walk(node):
                if (isinstance(inner, ast.Constant) and isinstance(inner.value, str) and
                        "\t" in inner.value and inner.value.startswith(VERBS)):
                    lines.append({"test": node.name, "line": inner.value})
    fixture = {
        "source": "tests/server/test_expert_server.py (data literals only)",
        "ready_lines": cases,
        "command_lines": lines,
    }
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "worker_protocol.json")
    with open(out, "w", encoding="utf-8") as target:
        json.dump(fixture, target, indent=1, sort_keys=True)
        target.write("\n")
    print(f"{len(cases)} ready lines, {len(lines)} command lines -> {out}")


if __name__ == "__main__":
    main()
