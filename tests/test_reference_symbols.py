"""The launcher names the reference's generator yields, against include/cumo_hip.h.

The reference's extension is generated: gen/cogen.rb evaluates gen/def/<type>.rb and then
gen/spec.rb, whose directives (binary "add", accum "sum", math "exp", store_from "Bit" ...)
each render one ERB template of gen/tmpl (gen/tmpl_bit first for Bit); the templates' host
sides declare the `cumo_*_kernel_launch` functions the device side has to define
(gen/erbpp2.rb:239-255 for how `c_func` / `c_iter` are spelled, gen/narray_def.rb:5-95 for
the directives, :181-197 for `store_from`). There is no Ruby here, so this file reads
spec.rb and the templates as text and expands them with a small translator for the handful
of Ruby constructs they use; where a construct is beyond it, BOTH branches are taken, so the
set of names can only grow. narray/{data,index,ndloop}.c are plain C and are scanned as is.

Every name found for SFloat, DFloat, Int32 and Bit must be declared in include/cumo_hip.h,
or fall under an entry of NOT_PROVIDED (whole templates that are outside this library's
scope, each with the reason). The test is skipped where the reference tree is absent."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = "/root/reference/ext/cumo/narray"
GEN = os.path.join(REF, "gen")

pytestmark = pytest.mark.skipif(not os.path.isdir(GEN), reason="the reference tree is not present on this machine")

TYPES = ("sfloat", "dfloat", "int32", "bit")

# Templates whose launchers this library does not provide: the part of the reference beside
# the array hot path (random numbers, histogram, sort, BLAS, cuDNN). A build of the whole
# extension on this library still needs these from elsewhere.
NOT_PROVIDED = {
    "rand": "random numbers (Philox generator): not on the elementwise / reduction path",
    "rand_norm": "random numbers: not on the path",
    "bincount": "histogram by scattered atomics: not on the path",
    "sort": "sorting (thrust/cub in the reference): not on the path",
    "sort_index": "sorting: not on the path",
    "median": "selection by sorting: not on the path",
    "qsort": "host quicksort template, no launcher of its own",
    "gemm": "dense contraction through the BLAS library: not on the path",
    "conv": "cuDNN", "conv_transpose": "cuDNN", "conv_grad_w": "cuDNN", "batch_norm": "cuDNN",
    "batch_norm_backward": "cuDNN", "fixed_batch_norm": "cuDNN", "pooling_forward": "cuDNN", "pooling_backward": "cuDNN",
}
# store_from sources the library provides launchers for: the four classes, plus Int64 (what the
# integer reductions and index arrays produce) and, into Bit only, UInt64 (what count_true
# produces). A `cumo_iter_<t>_store_<src>_kernel_launch` for any other source class (the
# narrow integers, unsigned, complex, RObject) belongs to a class outside this library.
STORE_SOURCES = {"bit", "dfloat", "sfloat", "int64", "int32", "numeric", "array"}


# ---------------------------------------------------------------------------------------
# a small Ruby-expression translator, enough for the conditions and names in the templates
# ---------------------------------------------------------------------------------------
class Name(str):
    """`c_func` is used both bare and as `c_func(:nodef)`."""
    def __call__(self, *a):
        return str(self)


class Untranslatable(Exception):
    pass


def ruby_to_py(e):
    e = e.strip()
    e = re.sub(r"%w\[([^\]]*)\]", lambda m: repr(m.group(1).split()), e)
    e = re.sub(r":([a-z_]+)\b(?!\s*=>)", r"'\1'", e) if re.search(r"\(:[a-z_]+\)", e) else e
    e = re.sub(r'#\{([^}]*)\}', lambda m: "{" + ruby_to_py(m.group(1)) + "}", e)
    e = re.sub(r'(?<![\w\'"])"((?:[^"\\]|\\.)*)"', lambda m: 'f"' + m.group(1) + '"' if "{" in m.group(1) else m.group(0), e)
    e = re.sub(r"([\w\.]+)\.include\?\s*\(?\s*('[^']*'|\"[^\"]*\"|\w+)\s*\)?", r"(\2 in \1)", e)
    m = re.fullmatch(r"\((.+?)\s\?\s(.+?)\s:\s(.+)\)", e)
    if m:
        e = "(%s if %s else %s)" % (m.group(2), m.group(1), m.group(3))
    e = e.replace("&&", " and ").replace("||", " or ")
    e = re.sub(r"!(?!=)", " not ", e)
    e = re.sub(r"\bnil\b", "None", e)
    e = re.sub(r"\btrue\b", "True", e)
    e = re.sub(r"\bfalse\b", "False", e)
    e = e.replace(".downcase", ".lower()").replace(".upcase", ".upper()")
    if re.search(r"::|\bdo\b|\.each|=>|\|", e):
        raise Untranslatable(e)
    return e


def ev(expr, ns):
    try:
        return eval(ruby_to_py(expr), {"__builtins__": {}}, ns)
    except Untranslatable:
        raise
    except Exception as exc:  # NameError for a helper the translator does not model, SyntaxError for Ruby it cannot read
        raise Untranslatable("%s (%s)" % (expr, exc))


UNKNOWN = "\u00a7"   # marks the output of a `<%= %>` that could not be evaluated


def render(text, ns):
    """ERB -> text. Control tags: if / unless / elsif / else / end, `<list>.each do |v|`,
    `v = <expr>`. A condition that cannot be evaluated takes every branch."""
    tokens = re.split(r"(<%=?.*?%>)", text, flags=re.S)
    # build a tree
    root = ("seq", [])
    stack = [root]

    def add(node):
        stack[-1][1].append(node)

    for tok in tokens:
        if tok.startswith("<%="):
            add(("expr", tok[3:-2].strip()))
        elif tok.startswith("<%"):
            code = tok[2:-2].strip()
            for stmt in [s.strip() for s in code.split(";") if s.strip()] if re.fullmatch(r"(end\s*;\s*)+end", code) else [code]:
                m = re.match(r"(.+?)\.each(?:_with_index)?\s+do\s*\|\s*(\w+(?:\s*,\s*\w+)*)\s*\|\s*(.*)$", stmt, flags=re.S)
                if m:
                    node = ("for", [], m.group(1), [v.strip() for v in m.group(2).split(",")])
                    add(node)
                    stack.append(node)
                    for rest in m.group(3).splitlines():   # assignments that follow the loop head in the same tag
                        if re.fullmatch(r"\s*\w+\s*=\s*[^=].*", rest):
                            add(("assign", rest.strip()))
                elif re.match(r"(if|unless)\b", stmt):
                    kw, cond = stmt.split(None, 1)
                    node = ("if", [], [[kw, cond, []]])
                    add(node)
                    stack.append(("branch", node[2][-1][2], node))
                elif re.match(r"elsif\b", stmt):
                    br = stack.pop()
                    br[2][2].append(["if", stmt.split(None, 1)[1], []])
                    stack.append(("branch", br[2][2][-1][2], br[2]))
                elif stmt == "else":
                    br = stack.pop()
                    br[2][2].append(["else", None, []])
                    stack.append(("branch", br[2][2][-1][2], br[2]))
                elif stmt == "end":
                    if len(stack) > 1:
                        stack.pop()
                elif re.fullmatch(r"\w+\s*=\s*[^=].*", stmt, flags=re.S):
                    add(("assign", stmt))
                else:
                    add(("code", stmt))
        elif tok:
            add(("text", tok))

    out = []

    def run(nodes, ns):
        for node in nodes:
            kind = node[0]
            if kind == "text":
                out.append(node[1])
            elif kind == "expr":
                try:
                    out.append(str(ev(node[1], ns)))
                except Untranslatable:
                    out.append(UNKNOWN)
            elif kind == "assign":
                var, expr = node[1].split("=", 1)
                try:
                    ns[var.strip()] = ev(expr, ns)
                except Untranslatable:
                    pass
            elif kind == "for":
                try:
                    values = list(ev(node[2], ns))
                except Untranslatable:
                    values = [UNKNOWN]
                for v in values:
                    names = node[3]
                    bound = dict(zip(names, v)) if len(names) > 1 and isinstance(v, (list, tuple)) else {names[0]: v}
                    run(node[1], dict(ns, **bound))
            elif kind == "if":
                taken = False
                for kw, cond, body in node[2]:
                    if kw == "else":
                        if not taken:
                            run(body, ns)
                        continue
                    try:
                        c = bool(ev(cond, ns))
                        if kw == "unless":
                            c = not c
                    except Untranslatable:
                        run(body, ns)       # unknown: this branch AND the ones after it
                        continue
                    if c and not taken:
                        run(body, ns)
                        taken = True

    run(root[1], ns)
    return "".join(out)


# ---------------------------------------------------------------------------------------
# gen/def/<type>.rb and gen/spec.rb
# ---------------------------------------------------------------------------------------
def type_flags(tname):
    ns = {}
    for line in open(os.path.join(GEN, "def", tname + ".rb")):
        m = re.match(r"\s*set\s+(\w+):\s*(.+?)\s*$", line)
        if m:
            v = m.group(2)
            ns[m.group(1)] = {"true": True, "false": False, "nil": None}.get(v, v.strip('"'))
    return ns


def spec_directives(flags):
    """(template, method name, kind, extra) for every directive of spec.rb that is live for
    this type. kind: 'method' (c_func = <type>_<name>), 'class_function' (<type>_s_<name>),
    'math' (<type>_math_s_<name>), 'store' (<type>_store_<name>)."""
    out = []
    live = [True]
    in_math = False
    block = []   # what each open `do` / `if` was
    for raw in open(os.path.join(GEN, "spec.rb")):
        line = raw.split("#", 1)[0].strip() if not re.search(r'"[^"]*#', raw) else raw.strip()
        if not line:
            continue
        m = re.match(r"if\s+(.+)$", line)
        if m and not re.search(r"\bif\b.*\bif\b", line):
            cond = bool(ev(m.group(1), flags)) if all(live) else False
            live.append(cond)
            block.append("if")
            continue
        if line == "else":
            outer = all(live[:-1])
            live[-1] = outer and not live[-1]
            continue
        if line.startswith("end"):
            if block:
                what = block.pop()
                if what == "if":
                    live.pop()
                elif what == "math":
                    in_math = False
            continue
        post = re.match(r"(.+?)\s+if\s+(.+)$", line)
        if post:
            if not ev(post.group(2), flags):
                continue
            line = post.group(1)
        if re.search(r"\bdo\b\s*$", line):
            block.append("math" if line.startswith("def_module") else "do")
            if line.startswith("def_module"):
                in_math = True
            line = re.sub(r"\s*do\s*$", "", line)
        if not all(live):
            continue
        local = re.fullmatch(r"(\w+)\s*=\s*(\w+)", line)   # `is_c = is_complex`
        if local:
            if local.group(2) in flags:
                flags[local.group(1)] = flags[local.group(2)]
            continue
        args = re.findall(r'"([^"]*)"', line)
        word = line.split()[0].split("(")[0]
        if word in ("binary", "binary2", "unary", "cond_binary", "cond_unary", "bit_count", "bit_count_cpu",
                    "accum_index", "accum_arg", "accum_binary", "unary2", "set2", "bit_reduce", "accum", "cum"):
            out.append((word, args[0], "method", {}))
        elif word == "pow":
            out.append(("pow", "pow", "method", {}))
        elif word in ("def_method", "def_singleton_method"):
            if args:
                out.append((args[1] if len(args) > 1 else args[0], args[0], "method", {}))
        elif word == "def_alloc_func":
            out.append((args[0], args[0], "method", {}))
        elif word == "def_module_function":
            out.append((args[1] if len(args) > 1 else args[0], args[0], "class_function", {}))
        elif word == "math" and in_math:
            n = re.search(r'"\s*,\s*(\d)', line)
            tmpl = args[1] if len(args) > 1 else {"1": "unary_s", "2": "binary_s", "3": "ternary_s"}[n.group(1) if n else "1"]
            out.append((tmpl, args[0], "math", {}))
        elif word == "store_from":
            out.append(("store_bit" if args[0] == "Bit" else "store_from", args[0].lower(), "store", {"type_name": args[0]}))
        elif word == "store_numeric":
            out.append(("store_numeric", "numeric", "store", {}))
        elif word == "store_array":
            out.append(("store_array", "array", "store", {}))
        elif word == "qsort":
            out.append(("qsort", "qsort", "method", {}))
    return out


def c_name(name):
    return name.replace("?", "_p").replace("!", "_bang").replace("=", "_set")


def expected_names(tname):
    flags = type_flags(tname)
    dirs = [os.path.join(GEN, d) for d in (("tmpl_bit", "tmpl") if tname == "bit" else ("tmpl",))]
    names = {}      # launcher name -> template
    for tmpl, meth, kind, extra in spec_directives(flags):
        path = next((os.path.join(d, tmpl + ".c") for d in dirs if os.path.exists(os.path.join(d, tmpl + ".c"))), None)
        if path is None:
            continue
        cn = c_name(meth)
        c_func = {"method": "%s_%s", "class_function": "%s_s_%s", "math": "%s_math_s_%s", "store": "%s_store_%s"}[kind] % (tname, cn)
        ns = dict(flags)
        ns.update(extra)
        ns.update(name=meth, c_name=cn, c_func=Name(c_func), c_iter="iter_" + c_func, opt_indexer_ndim=4)
        if kind == "store" and "type_name" not in extra:
            ns["type_name"] = flags["type_name"]
        text = render(open(path).read(), ns)
        for n in re.findall(r"\bcumo_[A-Za-z0-9_%s]*_kernel_launch\b" % UNKNOWN, text):
            if kind == "store" and meth not in STORE_SOURCES:
                continue
            names.setdefault(n, tmpl)
    return names


def plain_c_names():
    names = {}
    for f in ("data.c", "index.c", "ndloop.c"):
        for n in re.findall(r"\bcumo_[a-z0-9_]+_kernel_launch\b", open(os.path.join(REF, f)).read()):
            names.setdefault(n, f)
    return names


def declared():
    txt = ""
    for h in ("cumo_hip.h", "cumo_hip_ndloop.h"):
        txt += subprocess.run(["gcc", "-E", "-P", "-I", os.path.join(ROOT, "include"), os.path.join(ROOT, "include", h)],
                              check=True, stdout=subprocess.PIPE, text=True).stdout
    return set(re.findall(r"\b(cumo_[a-z0-9_]+)\s*\(", txt))


def test_translator_on_the_constructs_the_templates_use():
    ns = {"is_float": True, "type_name": "sfloat", "name": "sum", "c_iter": "iter_sfloat_sum", "c_func": Name("sfloat_sum")}
    t = ('<% ops = %w[sum prod] %><% (is_float ? ["","_nan"] : [""]).each do |nan| %><% [64,32].each do |i| %>'
         '<% unless type_name == \'robject\' %>//<% unless ops.include?(name) %>\nA_<%=name%><%=nan%>_int<%=i%>;\n<% else %>\n'
         'B_<%="cumo_#{c_iter}#{nan}_x"%>_<%=i%>_<%="#{c_func(:nodef)}"%>;<% end %>\n<% end %><% end;end %>')
    got = re.findall(r"[AB]_\w+", render(t, ns))
    assert got == ["B_cumo_iter_sfloat_sum_x_64_sfloat_sum", "B_cumo_iter_sfloat_sum_x_32_sfloat_sum",
                   "B_cumo_iter_sfloat_sum_nan_x_64_sfloat_sum", "B_cumo_iter_sfloat_sum_nan_x_32_sfloat_sum"]
    ns["name"] = "other"
    assert re.findall(r"[AB]_\w+", render(t, ns))[0] == "A_other_int64"
    # a condition beyond the translator takes both branches
    assert render("<% if Gem::Version.create(X) < 3 %>p<% else %>q<% end %>", {}) == "pq"


def test_spec_expansion_finds_the_known_names():
    s = expected_names("sfloat")
    for n in ("cumo_iter_sfloat_add_kernel_launch", "cumo_iter_sfloat_add_s_kernel_launch", "cumo_iter_sfloat_math_s_exp_kernel_launch",
              "cumo_sfloat_sum_nan_kernel_launch", "cumo_sfloat_argmax_nan_int32_kernel_launch", "cumo_iter_sfloat_store_bit_kernel_launch",
              "cumo_iter_sfloat_store_sfloat_stridx_kernel_launch", "cumo_sfloat_minmax_nan_kernel_launch", "cumo_iter_sfloat_gt_s_kernel_launch",
              "cumo_sfloat_maximum_nan_kernel_launch", "cumo_iter_sfloat_math_s_frexp_kernel_launch", "cumo_sfloat_cumsum_nan_kernel_launch"):
        assert n in s, n
    assert "cumo_dfloat_kahan_sum_kernel_launch" in expected_names("dfloat")
    assert "cumo_sfloat_kahan_sum_kernel_launch" not in s
    i = expected_names("int32")
    assert "cumo_iter_int32_left_shift_s_kernel_launch" in i and "cumo_int32_sum_nan_kernel_launch" not in i
    assert "cumo_iter_int32_math_s_exp_kernel_launch" not in i
    b = expected_names("bit")
    for n in ("cumo_iter_bit_store_bit_kernel_launch", "cumo_iter_bit_store_bit_contiguous_kernel_launch", "cumo_iter_bit_all_p_reduce_kernel_launch",
              "cumo_iter_bit_count_false_index_stride_kernel_launch", "cumo_iter_bit_store_array_contiguous_kernel_launch", "cumo_bit_where_kernel_launch"):
        assert n in b, n
    assert not any(UNKNOWN in n for t in TYPES for n in expected_names(t)), "a launcher name could not be expanded"


def test_every_reference_launcher_is_declared_or_listed_as_not_provided():
    have = declared()
    missing = {}
    counted = 0
    for t in TYPES:
        for n, tmpl in sorted(expected_names(t).items()):
            counted += 1
            if n in have or tmpl in NOT_PROVIDED:
                continue
            missing[n] = "gen/tmpl*/%s.c (%s)" % (tmpl, t)
    for n, f in sorted(plain_c_names().items()):
        counted += 1
        if n not in have:
            missing[n] = "narray/" + f
    assert counted > 450, counted
    assert not missing, "launchers of the reference with no declaration in include/cumo_hip.h:\n" + "\n".join("  %s  <- %s" % kv for kv in sorted(missing.items()))


def test_not_provided_table_is_not_stale():
    """An entry stays in NOT_PROVIDED only while the header really lacks its launchers."""
    have = declared()
    for t in TYPES:
        by_tmpl = {}
        for n, tmpl in expected_names(t).items():
            by_tmpl.setdefault(tmpl, []).append(n)
        for tmpl, ns in by_tmpl.items():
            if tmpl in NOT_PROVIDED:
                assert not all(n in have for n in ns), "%s is provided now: take it out of NOT_PROVIDED" % tmpl
