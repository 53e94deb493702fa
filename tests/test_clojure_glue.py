"""The Clojure glue under clojure/src cannot be executed here (no JVM).  What can be checked on
the text is checked: every file reads as balanced Clojure forms, every `ct_*` entry point it
invokes is declared in include/cortex_hip.h with exactly as many parameters as the call passes
arguments, each argument is coerced to the class that JNA marshals at the width the header declares, every TensorMath method of the reference's protocol is implemented with the protocol's
arity, and every entry point of the header is reachable from the glue."""
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
GLUE = sorted((ROOT / "clojure" / "src" / "cortex" / "compute" / "hip").glob("*.clj"))
HEADER = ROOT / "include" / "cortex_hip.h"

OPEN, CLOSE = "([{", ")]}"
PAIR = dict(zip(CLOSE, OPEN))


def read_forms(text: str):
    """A small Clojure reader: returns the top-level forms as nested lists of tokens.  Strings are
    kept as ('str', value); comments and whitespace are dropped.  Raises on unbalanced input."""
    pos, n = 0, len(text)
    stack = [[]]
    opened = []
    while pos < n:
        ch = text[pos]
        if ch in " \t\r\n,":
            pos += 1
        elif ch == ";":
            while pos < n and text[pos] != "\n":
                pos += 1
        elif ch == '"':
            end = pos + 1
            while text[end] != '"':
                end += 2 if text[end] == "\\" else 1
            stack[-1].append(("str", text[pos + 1:end]))
            pos = end + 1
        elif ch == "\\":                       # character literal
            m = re.match(r"\\(newline|space|tab|.)", text[pos:])
            stack[-1].append(m.group(0))
            pos += len(m.group(0))
        elif ch in OPEN:
            opened.append((ch, pos))
            new = [ch]
            stack[-1].append(new)
            stack.append(new)
            pos += 1
        elif ch in CLOSE:
            assert opened, f"unmatched {ch!r} at offset {pos}"
            o, where = opened.pop()
            assert o == PAIR[ch], f"{o!r} opened at offset {where} is closed by {ch!r} at offset {pos}"
            stack.pop()
            pos += 1
        elif ch == "^":                        # metadata: annotates the next form and is no form itself
            stack[-1].append(META)
            pos += 1
        elif ch in "'`~@#":                    # reader macros: prefix the next form; #{ and #( open collections
            if ch == "#" and pos + 1 < n and text[pos + 1] == "_":
                pos += 2
            else:
                pos += 1
        else:
            m = re.match(r"[^\s,;\"()\[\]{}]+", text[pos:])
            stack[-1].append(m.group(0))
            pos += len(m.group(0))
    assert not opened, f"{opened[-1][0]!r} opened at offset {opened[-1][1]} is never closed"
    return drop_metadata(stack[0])


META = object()


def drop_metadata(form):
    """Removes every metadata marker together with the form it introduces (^String, ^:const, ^{:doc ...})."""
    out, skip = [], False
    for item in form:
        if item is META:
            skip = True
        elif skip:
            skip = False
        else:
            out.append(drop_metadata(item) if isinstance(item, list) else item)
    return out


def walk(form):
    if isinstance(form, list):
        yield form
        for item in form:
            yield from walk(item)


def header_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    out = {}
    for m in re.finditer(r"\b(?:int|const char\*)\s+(ct_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        params = m.group(2).strip()
        out[m.group(1)] = 0 if params in ("", "void") else len([p for p in params.split(",") if p.strip()])
    return out


def glue_calls():
    """(file, function name, argument count) for every (call! "ct_..." ...) form."""
    calls = []
    for path in GLUE:
        for form in walk(read_forms(path.read_text())):
            if len(form) >= 3 and form[0] == "(" and form[1] == "call!" and isinstance(form[2], tuple):
                calls.append((path.name, form[2][1], len(form) - 3))
    return calls


def test_glue_files_exist_and_read_as_balanced_forms():
    names = {p.name for p in GLUE}
    assert {"ffi.clj", "driver.clj", "tensor_math.clj", "backend.clj", "optimize.clj", "context.clj"} <= names
    for path in GLUE:
        forms = read_forms(path.read_text())
        assert forms and forms[0][1] == "ns", path
        assert forms[0][2].startswith("cortex.compute.hip."), path


def test_every_native_call_matches_the_header():
    declared = header_functions()
    assert len(declared) > 50
    calls = glue_calls()
    assert len(calls) > 50
    for file, name, argc in calls:
        assert name in declared, f"{file}: {name} is not declared in include/cortex_hip.h"
        assert argc == declared[name], f"{file}: {name} is called with {argc} arguments, the header declares {declared[name]}"


def header_parameter_kinds():
    """Entry point -> the machine kind of each parameter: 'ptr', 'i32', 'i64', 'f64' or 'f32'."""
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    out = {}
    for m in re.finditer(r"\b(?:int|const char\*)\s+(ct_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        params = m.group(2).strip()
        kinds = []
        for p in ([] if params in ("", "void") else params.split(",")):
            p = p.strip()
            if "*" in p or "[" in p:
                kinds.append("ptr")
            elif re.match(r"(const\s+)?double\b", p):
                kinds.append("f64")
            elif re.match(r"(const\s+)?float\b", p):
                kinds.append("f32")
            elif re.match(r"(const\s+)?(u?int64_t|size_t)\b", p):
                kinds.append("i64")
            else:
                assert re.match(r"(const\s+)?(int|u?int32_t|unsigned|ct_[a-z_]+_t)\b", p), (m.group(1), p)
                kinds.append("i32")
        out[m.group(1)] = kinds
    return out


# How JNA marshals what each coercion of the glue produces (Integer -> 32 bits, Long -> 64 bits, Double -> a double,
# Pointer / Memory / ...ByReference / nil -> a pointer): the head of an argument form -> its machine kind.
COERCIONS = {
    "int": "i32", "dtype-code": "i32", "ffi/dtype-code": "i32", "op-code": "i32", "ffi/op-code": "i32",
    "bool->int": "i32", "ffi/bool->int": "i32",
    "long": "i64", "double": "f64", "float": "f32",
    "->ptr": "ptr", "dims": "ptr", ":handle": "ptr", "ffi/conv-desc->native": "ptr", "ffi/pool-desc->native": "ptr",
    "arg-indexes": "ptr", "when": "ptr",
}


def test_every_native_call_passes_the_headers_machine_types():
    """JNA picks the native width from the Java class of each argument, so an (int ...) where the header says
    int64_t, or a (long ...) where it says int, would put a wrong-sized value on the stack without any error.
    Every argument of every call is a coercion form whose result class is known, or a bare symbol (a handle, a
    pointer or a ...ByReference out-parameter): its kind must be the header's, parameter by parameter."""
    declared = header_parameter_kinds()
    checked = 0
    for path in GLUE:
        for form in walk(read_forms(path.read_text())):
            if not (len(form) >= 3 and form[0] == "(" and form[1] == "call!" and isinstance(form[2], tuple)):
                continue
            name, args = form[2][1], form[3:]
            for position, (arg, want) in enumerate(zip(args, declared[name])):
                if isinstance(arg, str):
                    assert not re.fullmatch(r"-?[0-9.]+", arg), f"{path.name}: {name} argument {position} is a bare number"
                    got = "ptr"
                else:
                    assert isinstance(arg, list) and arg[0] == "(", f"{path.name}: {name} argument {position}: {arg!r}"
                    assert arg[1] in COERCIONS, f"{path.name}: {name} argument {position} is built by {arg[1]!r}, whose class is unknown"
                    got = COERCIONS[arg[1]]
                assert got == want, f"{path.name}: {name} argument {position} is passed as {got}, the header declares {want}"
                checked += 1
    assert checked > 400


def header_pointee_types():
    """Entry point -> per parameter the C type a pointer parameter points to (None for values)."""
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    out = {}
    for m in re.finditer(r"\b(?:int|const char\*)\s+(ct_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        params = m.group(2).strip()
        types = []
        for p in ([] if params in ("", "void") else params.split(",")):
            pm = re.match(r"\s*(?:const\s+)?([A-Za-z_0-9]+)\s*(\*+)", p)
            types.append(pm.group(1) + pm.group(2)[1:] if pm else None)
        out[m.group(1)] = types
    return out


BY_REFERENCE = {"IntByReference.": {"int", "int32_t"}, "LongByReference.": {"size_t", "int64_t", "uint64_t"},
                "FloatByReference.": {"float"}, "PointerByReference.": {"void*"}}


def test_out_parameters_use_the_reference_class_of_the_pointee():
    """An out-parameter is a JNA ...ByReference object bound by an enclosing let: its class fixes how many bytes
    the library's store may write (an IntByReference under a size_t* would be overrun)."""
    pointees = header_pointee_types()
    checked = 0
    for path in GLUE:
        for top in read_forms(path.read_text()):
            bound = {}
            for form in walk(top):
                if len(form) >= 3 and form[0] == "(" and form[1] in ("let", "let*") and isinstance(form[2], list) and form[2][0] == "[":
                    pairs = form[2][1:]
                    for sym, init in zip(pairs[0::2], pairs[1::2]):
                        if isinstance(sym, str) and isinstance(init, list) and len(init) >= 2 and isinstance(init[1], str):
                            ctor = init[1].split(".")[-2] + "." if init[1].endswith("ByReference.") else None
                            if ctor:
                                bound[sym] = ctor
            for form in walk(top):
                if len(form) >= 3 and form[0] == "(" and form[1] == "call!" and isinstance(form[2], tuple):
                    name = form[2][1]
                    for position, (arg, pointee) in enumerate(zip(form[3:], pointees[name])):
                        if isinstance(arg, str) and arg in bound:
                            assert pointee in BY_REFERENCE[bound[arg]], \
                                f"{path.name}: {name} argument {position} is a {bound[arg][:-1]}, the header declares {pointee}*"
                            checked += 1
    assert checked >= 10


LAYOUT_PROBE = r"""
#include <stddef.h>
#include <stdio.h>
#include "cortex_hip.h"
int main(void) {
  printf("dims %zu %zu %zu %zu %zu\n", sizeof(ct_dims), offsetof(ct_dims, ndim), offsetof(ct_dims, shape),
         offsetof(ct_dims, strides), offsetof(ct_dims, index));
  printf("pool %zu %zu %zu %zu %zu %zu %zu %zu\n", sizeof(ct_pool_desc), offsetof(ct_pool_desc, kernel_width),
         offsetof(ct_pool_desc, kernel_height), offsetof(ct_pool_desc, pad_x), offsetof(ct_pool_desc, pad_y),
         offsetof(ct_pool_desc, stride_x), offsetof(ct_pool_desc, stride_y), offsetof(ct_pool_desc, pool_op));
  printf("conv %zu %zu %zu %zu %zu %zu %zu %zu %zu\n", sizeof(ct_conv_desc), offsetof(ct_conv_desc, in_channels),
         offsetof(ct_conv_desc, out_channels), offsetof(ct_conv_desc, kernel_width), offsetof(ct_conv_desc, kernel_height),
         offsetof(ct_conv_desc, pad_x), offsetof(ct_conv_desc, pad_y), offsetof(ct_conv_desc, stride_x),
         offsetof(ct_conv_desc, stride_y));
  printf("max_dims %d\n", CT_MAX_DIMS);
  return 0;
}
"""


def test_struct_layouts_written_by_hand_are_the_compilers(tmp_path):
    """ffi.clj fills ct_dims, ct_pool_desc and ct_conv_desc byte by byte into raw memory: the sizes and offsets
    it uses are compared with what the C compiler makes of the header, field by field and in field order."""
    import subprocess
    src = tmp_path / "layout.c"
    src.write_text(LAYOUT_PROBE)
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c99", "-I", str(HEADER.parent), str(src), "-o", str(exe)], check=True)
    probe = {line.split()[0]: [int(v) for v in line.split()[1:]]
             for line in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines()}
    text = (ROOT / "clojure" / "src" / "cortex" / "compute" / "hip" / "ffi.clj").read_text()
    const = lambda name: int(re.search(r"\(def \^:const " + re.escape(name) + r" (\d+)\)", text).group(1))
    assert [const("dims-byte-size"), 0, const("dims-shape-offset"), const("dims-strides-offset"), const("dims-index-offset")] == probe["dims"]
    assert const("ct-max-dims") == probe["max_dims"][0]
    assert "(.setInt mem 0 (int (count shape)))" in text          # ndim at offset 0
    forms = read_forms(text)

    def descriptor(defn_name):
        """(bytes allocated, [(offset, field symbol)] in the order written) of a `(doto (Memory. n) (.setInt off x) ...)`."""
        body = [f for f in forms if f[:3] == ["(", "defn", defn_name]][0]
        doto = [f for f in walk(body) if f[:2] == ["(", "doto"]][0]
        size = int(doto[2][2])
        writes = []
        for f in doto[3:]:
            assert f[1] == ".setInt", f
            value = f[3]
            writes.append((int(f[2]), value[2] if value[1] == "int" else value[-1]))
        return size, writes

    size, writes = descriptor("pool-desc->native")
    assert [size] + [off for off, _ in writes] == probe["pool"]
    assert [name for _, name in writes] == ["kernel-width", "kernel-height", "pad-x", "pad-y", "stride-x", "stride-y", "pool-op"]
    size, writes = descriptor("conv-desc->native")
    assert [size] + [off for off, _ in writes] == probe["conv"]
    assert [name for _, name in writes] == ["in-channels", "out-channels", "kernel-width", "kernel-height", "pad-x", "pad-y",
                                            "stride-x", "stride-y"]
    # the ctypes mirror used by the Python side
    import ctypes as C
    from cortex_amd import capi
    assert [C.sizeof(capi.CtDims), capi.CtDims.ndim.offset, capi.CtDims.shape.offset, capi.CtDims.strides.offset,
            capi.CtDims.index.offset] == probe["dims"]


# keyword of the reference's API -> enumerator suffix of the header, per table
ENUM_NAMES = {
    ("datatype->code", "CT_"): {"byte": "I8", "short": "I16", "int": "I32", "long": "I64", "float": "F32", "double": "F64",
                                "ubyte": "U8"},
    ("unary-op->code", "CT_UOP_"): {"floor": "FLOOR", "ceil": "CEIL", "round": "ROUND", "-": "NEGATE", "tanh": "TANH",
                                    "logistic": "LOGISTIC", "exp": "EXP", "sqrt": "SQRT", "noop": "NOOP"},
    ("binary-op->code", "CT_BOP_"): {"+": "ADD", "-": "SUB", "*": "MUL", "/": "DIV", "min": "MIN", "max": "MAX",
                                     "bit-and": "BIT_AND", "bit-xor": "BIT_XOR", "eq": "EQ", ">": "GT", ">=": "GE", "<": "LT",
                                     "<=": "LE"},
    ("ternary-op->code", "CT_TOP_"): {"select": "SELECT"},
    ("reduce-op->code", "CT_ROP_"): {"max": "MAX", "min": "MIN", "sum": "SUM", "mean": "MEAN", "magnitude": "MAGNITUDE",
                                     "magnitude-squared": "MAGNITUDE_SQUARED"},
    ("activation-op->code", "CT_ACT_"): {"logistic": "LOGISTIC", "tanh": "TANH", "relu": "RELU"},
    ("pool-op->code", "CT_POOL_"): {"max": "MAX", "avg": "AVG", "avg-exc-pad": "AVG_EXC_PAD"},
    ("copy-kind", "CT_COPY_"): {"host->device": "HOST_TO_DEVICE", "device->host": "DEVICE_TO_HOST",
                                "device->device": "DEVICE_TO_DEVICE"},
}


def test_code_tables_are_the_headers_enumerators():
    """The keyword -> code maps of ffi.clj, and the tables of the Python side, against the enumerators of the header:
    same keys, same numbers."""
    header = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    enumerators = {m.group(1): int(m.group(2)) for m in re.finditer(r"\b(CT_[A-Z0-9_]+)\s*=\s*(\d+)", header)}
    forms = read_forms((ROOT / "clojure" / "src" / "cortex" / "compute" / "hip" / "ffi.clj").read_text())
    from cortex_amd import capi
    python_tables = {"datatype->code": capi.DTYPE_CODES, "unary-op->code": capi.UNARY_OPS, "binary-op->code": capi.BINARY_OPS,
                     "ternary-op->code": capi.TERNARY_OPS, "reduce-op->code": capi.REDUCE_OPS,
                     "activation-op->code": capi.ACTIVATION_OPS, "pool-op->code": capi.POOL_OPS,
                     "copy-kind": {"host->device": capi.COPY_H2D, "device->host": capi.COPY_D2H, "device->device": capi.COPY_D2D}}
    for (table, prefix), names in ENUM_NAMES.items():
        form = [f for f in forms if f[:3] == ["(", "def", table]][0]
        literal = [x for x in form[3:] if isinstance(x, list) and x[0] == "{"][0][1:]
        glue = {k.lstrip(":"): int(v) for k, v in zip(literal[0::2], literal[1::2])}
        want = {key: enumerators[prefix + suffix] for key, suffix in names.items()}
        assert glue == want, (table, glue, want)
        assert python_tables[table] == want, (table, python_tables[table], want)
        # and no enumerator of that family is left without a keyword
        family = {n for n in enumerators if n.startswith(prefix) and (prefix != "CT_" or re.fullmatch(r"CT_[IUF]\d+", n))}
        assert family == {prefix + suffix for suffix in names.values()}, (table, family)
    assert capi.DISTRIBUTIONS == {"gaussian": enumerators["CT_DIST_GAUSSIAN"], "flat": enumerators["CT_DIST_FLAT"]}
    tm = (ROOT / "clojure" / "src" / "cortex" / "compute" / "hip" / "tensor_math.clj").read_text()
    assert re.search(r":gaussian \[%d " % enumerators["CT_DIST_GAUSSIAN"], tm) and re.search(r":flat \[%d " % enumerators["CT_DIST_FLAT"], tm)


DEFINERS = {"def", "defn", "defn-", "defmacro", "defmulti", "defonce", "declare", "defrecord", "deftype", "defprotocol"}


def namespace_of(forms):
    """(name, {alias: namespace}, {referred symbol: namespace}) of a file's ns form."""
    ns = forms[0]
    aliases, refers = {}, {}
    for clause in ns[3:]:
        if isinstance(clause, list) and len(clause) > 1 and clause[1] == ":require":
            for spec in clause[2:]:
                if not (isinstance(spec, list) and spec[0] == "["):
                    continue
                target, rest = spec[1], spec[2:]
                for key, value in zip(rest[0::2], rest[1::2]):
                    if key == ":as":
                        aliases[value] = target
                    elif key == ":refer" and isinstance(value, list):
                        for sym in value[1:]:
                            refers[sym] = target
    return ns[2], aliases, refers


def definitions(forms):
    """Names a file defines at top level -> whether they are private; protocols also define their methods and
    records their constructor functions."""
    out = {}
    for form in forms:
        if not (isinstance(form, list) and len(form) > 2 and form[0] == "(" and form[1] in DEFINERS):
            continue
        names = form[2:] if form[1] == "declare" else [form[2]]
        for name in names:
            if not isinstance(name, str):
                continue
            out[name] = form[1] == "defn-"
            if form[1] in ("defrecord", "deftype"):
                out["->" + name] = False
                out["map->" + name] = False
            if form[1] == "defprotocol":
                for method in form[3:]:
                    if isinstance(method, list) and method[0] == "(" and isinstance(method[1], str):
                        out[method[1]] = False
    return out


def symbols_with_namespace(form):
    for item in form:
        if isinstance(item, list):
            yield from symbols_with_namespace(item)
        elif isinstance(item, str) and "/" in item and not item.startswith((":", "\\")) and len(item) > 1:
            alias, _, name = item.partition("/")
            if alias and name:
                yield alias, name


def test_symbols_of_other_namespaces_exist_where_they_are_looked_up():
    """No compiler has seen these files: every `alias/name` and every :refer that points into another file of the
    glue must name something that file defines publicly, and, where the reference's sources are at hand, the same
    for what points into the reference's namespaces (protocols, multimethods, helper functions)."""
    files = {}
    for path in GLUE:
        forms = read_forms(path.read_text())
        name, aliases, refers = namespace_of(forms)
        files[name] = (path, forms, aliases, refers, definitions(forms))
    reference_root = Path("/root/reference/src")
    reference_cache = {}

    def defined_in(namespace):
        if namespace in files:
            return {n for n, private in files[namespace][4].items() if not private}
        source = reference_root / (namespace.replace(".", "/").replace("-", "_") + ".clj")
        if not source.exists():
            return None                      # a library that is not vendored, or no reference on this machine
        if namespace not in reference_cache:
            reference_cache[namespace] = {n for n, private in definitions(read_forms(source.read_text())).items() if not private}
        return reference_cache[namespace]

    checked = 0
    for name, (path, forms, aliases, refers, _own) in files.items():
        for sym, target in refers.items():
            known = defined_in(target)
            if known is not None:
                assert sym in known, f"{path.name}: refers to {target}/{sym}, which {target} does not define"
                checked += 1
        for alias, sym in set(symbols_with_namespace(forms[1:])):
            if alias not in aliases:
                continue                     # a Java class with a static member, or a fully qualified name
            known = defined_in(aliases[alias])
            if known is not None:
                assert sym in known, f"{path.name}: {alias}/{sym} is not defined in {aliases[alias]}"
                checked += 1
    assert checked > 20


def test_every_entry_point_is_bound():
    declared = set(header_functions())
    text = "".join(p.read_text() for p in GLUE)
    named = set(re.findall(r'"(ct_[a-z0-9_]+)"', text))
    assert declared - named == set(), sorted(declared - named)


def reference_protocol_arities():
    """Method name -> parameter count of cortex.tensor.math/TensorMath, read from the reference when it
    is present (it is not on the GPU box); the stored copy of the counts otherwise."""
    ref = Path("/root/reference/src/cortex/tensor/math.clj")
    if not ref.exists():
        return None
    proto = [f for f in read_forms(ref.read_text()) if f[:2] == ["(", "defprotocol"]][0]
    return {m[1]: len(m[2]) - 1 for m in proto if isinstance(m, list) and m[0] == "(" and isinstance(m[2], list)}


# name -> number of parameters (stream included), src/cortex/tensor/math.clj:11-252
TENSOR_MATH = {
    "assign-constant!": 5, "assign!": 6, "unary-accum!": 6, "unary-op!": 8, "binary-accum-constant!": 8,
    "binary-op-constant!": 10, "binary-accum!": 11, "binary-op!": 11, "ternary-op!": 14, "ternary-op-constant!": 13,
    "ternary-op-constant-constant!": 11, "unary-reduce!": 7, "gemm!": 14, "gemv!": 12,
    "batch-normalize-eltwise!": 10, "batch-normalize-spatial!": 11, "batch-normalize-update-and-apply-eltwise!": 13,
    "batch-normalize-update-and-apply-spatial!": 14, "batch-normalize-gradients-eltwise!": 14,
    "batch-normalize-gradients-spatial!": 15, "activation-gradient!": 9, "softmax-eltwise!": 5, "softmax-spatial!": 5,
    "convolution-descriptor": 10, "choose-convolution-algorithms": 9, "convolution-forward!": 12,
    "convolution-backward-weights!": 12, "convolution-backward-data!": 12, "pooling-descriptor": 10,
    "pooling-forward!": 7, "pooling-backward!": 11, "rand!": 4, "lrn-descriptor": 5, "lrn-forward!": 6,
    "lrn-backward!": 10,
}


def test_stored_protocol_arities_are_the_references():
    live = reference_protocol_arities()
    if live is None:
        pytest.skip("the reference is not mounted here")
    assert live == TENSOR_MATH


def test_tensor_math_is_extended_with_the_protocols_arities():
    forms = read_forms((ROOT / "clojure/src/cortex/compute/hip/tensor_math.clj").read_text())
    ext = [f for f in forms if f[:3] == ["(", "extend-type", "HipStream"]]
    assert len(ext) == 1
    assert ext[0][3] == "tm/TensorMath"
    methods = {m[1]: len(m[2]) - 1 for m in ext[0][4:] if isinstance(m, list) and m[0] == "("}
    assert methods == TENSOR_MATH


def test_driver_protocols_are_implemented():
    text = (ROOT / "clojure/src/cortex/compute/hip/driver.clj").read_text()
    for method in ("get-devices", "allocate-host-buffer-impl", "memory-info-impl", "create-stream-impl",
                   "allocate-device-buffer-impl", "allocate-rand-buffer-impl", "sub-buffer-impl", "alias?",
                   "partially-alias?", "copy-host->device", "copy-device->host", "copy-device->device", "memset",
                   "create-event", "sync-event", "wait-for-event", "get-driver", "get-device"):
        assert re.search(r"\(" + re.escape(method) + r"\s+\[", text), method
    opt = (ROOT / "clojure/src/cortex/compute/hip/optimize.clj").read_text()
    for key in ("[:hip :adam]", "[:hip :adadelta]", "[:hip :sgd]"):
        assert "(defmethod create-optimizer " + key in opt
