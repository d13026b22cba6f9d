"""
Reads the op descriptions of the reference's returnn/native_op.py as TEXT: the file is parsed with :mod:`ast` and the
class attributes ``in_info``, ``out_info``, ``c_fw_code``, ``c_bw_code``, ``c_extra_support_code``, ``code_version`` are
evaluated by a tiny evaluator that knows literals, names of module-level literals, ``copy.copy(x)``, ``Class.attr``,
subscripts and ``x.update({...})``; a ``grad_input_map`` method that returns some of its arguments is read as the tuple
of their positions.  Nothing of the reference is imported or executed, and nothing is written into this repository: the
descriptions are handed to the HIP op loader with a temporary cache directory, to check that the reference's op sources
compile against this package's dialect header.
"""

from __future__ import annotations

import ast
import copy
import os
from typing import Any, Dict

REFERENCE_NATIVE_OP = "/root/reference/returnn/native_op.py"
FIELDS = ("in_info", "out_info", "c_fw_code", "c_bw_code", "c_extra_support_code", "code_version", "grad_input_map")


class NotStatic(Exception):
    """an expression the evaluator does not cover"""


def _eval(node: ast.AST, module_env: Dict[str, Any], classes: Dict[str, Dict[str, Any]], local: Dict[str, Any]):
    try:
        return ast.literal_eval(node)
    except (ValueError, TypeError, SyntaxError):
        pass
    if isinstance(node, ast.Name):
        if node.id in local:
            return local[node.id]
        if node.id in module_env:
            return module_env[node.id]
        raise NotStatic(node.id)
    if isinstance(node, ast.Attribute) and isinstance(node.value, ast.Name) and node.value.id in classes:
        fields = classes[node.value.id]
        if node.attr in fields:
            return fields[node.attr]
        raise NotStatic("%s.%s" % (node.value.id, node.attr))
    if isinstance(node, ast.Subscript):
        base = _eval(node.value, module_env, classes, local)
        key = _eval(node.slice, module_env, classes, local)
        return base[key]
    if isinstance(node, ast.Call) and isinstance(node.func, ast.Attribute) and isinstance(node.func.value, ast.Name):
        if node.func.value.id == "copy" and node.func.attr in ("copy", "deepcopy") and len(node.args) == 1:
            return copy.deepcopy(_eval(node.args[0], module_env, classes, local))
    if isinstance(node, ast.Dict):
        return {
            _eval(k, module_env, classes, local): _eval(v, module_env, classes, local) for k, v in zip(node.keys, node.values)
        }
    if isinstance(node, ast.Tuple):
        return tuple(_eval(v, module_env, classes, local) for v in node.elts)
    raise NotStatic(ast.dump(node)[:80])


def read_descriptions(path: str = REFERENCE_NATIVE_OP):
    """
    :return: ``{class name: {field: value}}`` for every class that has forward code, and ``{class name: reason}`` for
        those whose fields could not be evaluated statically
    """
    tree = ast.parse(open(path).read())
    module_env: Dict[str, Any] = {}
    classes: Dict[str, Dict[str, Any]] = {}
    skipped: Dict[str, str] = {}
    for node in tree.body:
        if isinstance(node, ast.Assign) and len(node.targets) == 1 and isinstance(node.targets[0], ast.Name):
            try:
                module_env[node.targets[0].id] = ast.literal_eval(node.value)
            except (ValueError, TypeError, SyntaxError):
                pass
            continue
        if not isinstance(node, ast.ClassDef):
            continue
        local: Dict[str, Any] = {}
        problem = None
        for st in node.body:
            try:
                if isinstance(st, ast.Assign) and len(st.targets) == 1 and isinstance(st.targets[0], ast.Name):
                    if st.targets[0].id in FIELDS:
                        local[st.targets[0].id] = _eval(st.value, module_env, classes, local)
                elif isinstance(st, ast.FunctionDef) and st.name == "grad_input_map":
                    names = [a.arg for a in st.args.args][1:]  # without cls
                    returns = [b for b in st.body if isinstance(b, ast.Return)]
                    if len(returns) != 1 or not isinstance(returns[0].value, ast.Tuple):
                        raise NotStatic("grad_input_map body")
                    local["grad_input_map"] = tuple(names.index(e.id) for e in returns[0].value.elts)
                elif (
                    isinstance(st, ast.Expr)
                    and isinstance(st.value, ast.Call)
                    and isinstance(st.value.func, ast.Attribute)
                    and st.value.func.attr == "update"
                    and isinstance(st.value.func.value, ast.Name)
                    and st.value.func.value.id in FIELDS
                    and len(st.value.args) == 1
                ):
                    local[st.value.func.value.id].update(_eval(st.value.args[0], module_env, classes, local))
            except (NotStatic, KeyError) as exc:
                problem = "%s: %r" % (type(exc).__name__, exc.args[0] if exc.args else "")
                break
        if problem:
            skipped[node.name] = problem
            continue
        if local.get("c_fw_code"):
            if all(k in local for k in ("in_info", "out_info")):
                classes[node.name] = local
            else:
                skipped[node.name] = "no in_info/out_info in the class body"
    return classes, skipped


def as_description(name: str, fields: Dict[str, Any]):
    """A plain object with the attributes the op loader reads."""
    return type(name, (), dict(fields))


def available() -> bool:
    return os.path.exists(REFERENCE_NATIVE_OP)
