"""What can be said of the kernels without a device.

The launches in `dlgo_amd/kernels/ops.py` against the `extern "C"` declarations they call, read from the sources:
the number of arguments, and for every argument whose kind can be told from the call's text (a pointer, a stream, a
64-bit integer, a float) that the C parameter at its place is of that kind.  ctypes checks none of this without
declared argument types: a call with one argument too few, or a 64-bit count passed as a plain int, runs and reads
garbage.  Then what the libraries decide on the host alone: which product kernel a shape gets, how the decode
attention splits a sequence's pages, which widths the norm's hand-off covers, and what the launchers refuse before
they touch a device.  These need the compiler (the libraries are built at first use) but no GPU."""
import ast
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
CSRC = ROOT / "dlgo_amd" / "csrc"
OPS = ROOT / "dlgo_amd" / "kernels" / "ops.py"

DECL = re.compile(r'extern\s+"C"\s+(?P<ret>[\w\s\*]+?)\s*\b(?P<name>dlgo_\w+)\s*\((?P<params>[^)]*)\)\s*\{', re.S)


def kind_of(param: str) -> str:
    """'ptr', 'i64', 'f32', 'f64' or 'i32' for one C parameter declaration."""
    text = " ".join(param.split())
    if "*" in text or re.search(r"\bhipStream_t\b", text):
        return "ptr"
    words = text.split()[:-1]                      # without the parameter's name
    type_ = " ".join(w for w in words if w != "const")
    table = {"int": "i32", "int32_t": "i32", "unsigned": "i32", "unsigned int": "i32", "uint32_t": "i32",
             "long long": "i64", "int64_t": "i64", "unsigned long long": "i64", "uint64_t": "i64", "size_t": "i64",
             "float": "f32", "double": "f64"}
    assert type_ in table, f"unknown parameter type {text!r}"
    return table[type_]


def declarations():
    found = {}
    for path in sorted(CSRC.glob("*.hip")):
        for m in DECL.finditer(path.read_text()):
            params = [p for p in (q.strip() for q in m.group("params").split(",")) if p and p != "void"]
            found[m.group("name")] = (path.name, " ".join(m.group("ret").split()), [kind_of(p) for p in params], params)
    return found


def kind_of_argument(node: ast.AST):
    """What the text of an argument says about its kind, or None where it says nothing (a name, a sum)."""
    if isinstance(node, ast.Call):
        f = node.func
        name = f.attr if isinstance(f, ast.Attribute) else (f.id if isinstance(f, ast.Name) else "")
        return {"_ptr": "ptr", "_stream": "ptr", "c_void_p": "ptr", "byref": "ptr", "c_longlong": "i64", "c_ulonglong": "i64",
                "c_float": "f32", "c_double": "f64", "int": "i32", "c_int": "i32", "dtype_code": "i32", "_rows": "i32",
                "len": "i32"}.get(name)
    if isinstance(node, ast.Constant) and isinstance(node.value, (int, bool)):
        return "i32"
    return None


def tuple_lengths(func: ast.AST, name: str):
    """The tuples assigned to `name` inside a function, as lists of their elements."""
    out = []
    for node in ast.walk(func):
        if isinstance(node, ast.Assign) and any(isinstance(t, ast.Name) and t.id == name for t in node.targets):
            if isinstance(node.value, ast.Tuple):
                out.append(node.value.elts)
    return out


def calls():
    tree = ast.parse(OPS.read_text())
    found = []
    for func in [n for n in ast.walk(tree) if isinstance(n, (ast.FunctionDef, ast.AsyncFunctionDef))]:
        # names that stand for entry points: `fn = lib.dlgo_a if tiled else lib.dlgo_b` (the nearest assignment above a call counts)
        stand_ins = {}
        for node in ast.walk(func):
            if isinstance(node, ast.Assign) and len(node.targets) == 1 and isinstance(node.targets[0], ast.Name):
                names = {a.attr for a in ast.walk(node.value) if isinstance(a, ast.Attribute) and a.attr.startswith("dlgo_")}
                if names and not any(isinstance(c, ast.Call) and isinstance(c.func, ast.Attribute) and c.func.attr.startswith("dlgo_")
                                     for c in ast.walk(node.value)):
                    stand_ins.setdefault(node.targets[0].id, []).append((node.lineno, names))
        for node in ast.walk(func):
            if not isinstance(node, ast.Call):
                continue
            if isinstance(node.func, ast.Attribute) and node.func.attr.startswith("dlgo_"):
                entry_points = [node.func.attr]
            elif isinstance(node.func, ast.Name) and node.func.id in stand_ins:
                before = [(line, names) for line, names in stand_ins[node.func.id] if line <= node.lineno]
                entry_points = sorted(max(before, key=lambda ln: ln[0])[1])      # the assignment nearest above the call
            else:
                continue
            if True:
                args = []
                for a in node.args:
                    if isinstance(a, ast.Starred):
                        assert isinstance(a.value, ast.Name), f"line {node.lineno}: a starred argument that is no name"
                        tuples = tuple_lengths(func, a.value.id)
                        assert tuples and len({len(t) for t in tuples}) == 1, \
                            f"line {node.lineno}: *{a.value.id} is not a tuple of one length in {func.name}"
                        # every assignment must agree on the kinds that can be told
                        for i in range(len(tuples[0])):
                            kinds = {kind_of_argument(t[i]) for t in tuples} - {None}
                            assert len(kinds) <= 1, f"line {node.lineno}: *{a.value.id}[{i}] has kinds {kinds}"
                            args.append(kinds.pop() if kinds else None)
                    else:
                        args.append(kind_of_argument(a))
                assert not node.keywords
                found.extend((name, node.lineno, args) for name in entry_points)
    return found


def test_every_entry_point_is_declared_once_with_known_types():
    decl = declarations()
    assert len(decl) >= 25
    for name, (_, ret, kinds, _) in decl.items():
        assert ret in ("const char*", "int", "long long", "void"), (name, ret)
    # the entry point for callers that cannot allocate is declared in a header of its own as well
    assert "dlgo_argmax_noalloc" in decl and "dlgo_argmax_noalloc" in (CSRC / "sampling.h").read_text()


def test_the_launches_pass_what_the_declarations_take():
    decl = declarations()
    seen = calls()
    assert len(seen) >= 25
    for name, line, args in seen:
        assert name in decl, f"ops.py:{line} calls {name}, which no source declares"
        _, _, kinds, params = decl[name]
        assert len(args) == len(kinds), f"ops.py:{line}: {name} takes {len(kinds)} arguments, the call passes {len(args)}"
        for i, (got, want) in enumerate(zip(args, kinds)):
            if got is not None:
                assert got == want, f"ops.py:{line}: argument {i + 1} of {name} is passed as {got}, declared `{params[i]}`"
            else:
                # what the text does not tell may be a plain int only: pointers, 64-bit integers and floats are wrapped
                assert want == "i32", f"ops.py:{line}: argument {i + 1} of {name} (`{params[i]}`) must be wrapped for ctypes"


def test_functions_that_return_a_message_are_told_so():
    """`_lib` sets the return type of every function that returns an error message: one that it misses would hand back
    the low half of a pointer."""
    decl = declarations()
    text = OPS.read_text()
    listed = set(re.findall(r'"(dlgo_\w+)"', text[text.index("def _lib("):text.index("return lib", text.index("def _lib("))]))
    called = {name for name, _, _ in calls()}
    for name in called:
        if decl[name][1] == "const char*":
            assert name in listed, f"{name} returns a message but `_lib` does not set its return type"
        else:
            assert name not in listed, f"{name} returns {decl[name][1]}, not a message"


def test_the_choice_of_product_kernel_is_made_on_the_host(monkeypatch):
    """The rules that choose between the streamed and the tiled products count bytes, blocks and rows and ask the
    library's own planning functions, none of which touches a device: the table that the GPU test checks together with
    the products' results holds here too, for tensors that have a shape and nothing else, given 256 compute units."""
    import torch

    from dlgo_amd.kernels import ops
    from test_kernels_gpu import CHOICES
    monkeypatch.setattr(ops, "_cus", {0: 256})
    for n, k, t, streamed in CHOICES:
        w = torch.empty(n, k, dtype=torch.bfloat16, device="meta")
        assert ops.gemm_streams(w, t) is streamed, (n, k, t)
    # float32 rows are twice as long: the same widths fall on the other side of a rule
    w = torch.empty(2048, 4096, dtype=torch.float32, device="meta")
    assert ops.gemm_streams(w, 8) is ops.gemm_streams(torch.empty(2048, 8192, dtype=torch.bfloat16, device="meta"), 8)


def test_the_decode_attention_plans_its_splits_within_the_pages():
    """How many blocks share a sequence's pages in a step of single tokens is planned on the host from counts alone:
    for every shape there is at least one block, never more blocks than the longest sequence may have pages, and a
    step with many sequences does not split at all without long sequences to balance."""
    import ctypes

    from dlgo_amd.kernels import build
    for head_dim in (64, 128):
        lib = build.load("attention", (("HEAD_DIM", head_dim),))
        lib.dlgo_attention_decode_splits.restype = ctypes.c_int
        for n_seq in (1, 2, 8, 31, 64, 300):
            for n_heads, n_kv in ((32, 8), (24, 8), (6, 3), (40, 40), (64, 2)):
                for pages in (1, 3, 33, 64, 512, 2048):
                    for fused in (0, 1):
                        for variant in (0, 1):
                            s = lib.dlgo_attention_decode_splits(n_seq, n_heads, n_kv, pages, fused, variant)
                            assert 1 <= s <= pages, (head_dim, n_seq, n_heads, n_kv, pages, fused, variant, s)
                            if n_seq * n_kv >= 256 and pages <= 64:
                                assert s == 1, (head_dim, n_seq, n_heads, n_kv, pages, fused, variant, s)


def test_the_norm_hand_off_of_few_rows_knows_its_width():
    """A streamed product that leaves a norm keeps a share of every row's sum of squares per block of weight rows, and
    the product that applies the norm reads as many: beyond the widths those shares cover (256 of them), both say no,
    so that a model of hidden size 5,120 or 8,192 takes the norm kernel instead of a hand-off that cannot hold it."""
    import torch

    from dlgo_amd.kernels import ops

    def w(n, k):
        return torch.empty(n, k, dtype=torch.bfloat16, device="meta")
    for width in (2048, 3072, 4096):
        assert ops.streams_few_rows(w(width, width), 8, ops.ROLE_LEAVES_NORM), width
        assert ops.streams_few_rows(w(4 * width, width), 8, ops.ROLE_APPLIES_NORM), width
    for width in (5120, 8192):
        assert ops.streams_few_rows(w(width, width), 8, ops.ROLE_PLAIN), width
        assert not ops.streams_few_rows(w(width, width), 8, ops.ROLE_LEAVES_NORM), width
        assert not ops.streams_few_rows(w(4 * width, width), 8, ops.ROLE_APPLIES_NORM), width
    assert not ops.streams_few_rows(w(2048, 2048), 17, ops.ROLE_PLAIN)       # more rows than the streamed kernels take
    assert not ops.streams_few_rows(w(2048, 2040), 8, ops.ROLE_PLAIN)        # weight rows that are no whole kilobytes


def test_launchers_refuse_what_their_kernels_do_not_take():
    """Argument checks of the launchers come before anything touches a device, so the refusals can be read here: each
    names what was wrong."""
    import ctypes

    from dlgo_amd.kernels import build
    null, i64 = ctypes.c_void_p(0), ctypes.c_longlong
    rope = build.load("rope_kv")
    rope.dlgo_rope_kv.restype = ctypes.c_char_p

    def rope_kv(hd=64, rot=64, ld=None, n_heads=4, n_kv=2, write_kv=0):
        ld = (n_heads + 2 * n_kv) * hd if ld is None else ld
        return rope.dlgo_rope_kv(null, 1, 3, ld, n_heads, n_kv, hd, rot, 0, null, null, 0, null, null, null, null, 0, null, i64(0),
                                 i64(0), write_kv, null, 0, i64(0), 0, 0, 0, null)
    assert b"rotated width" in rope_kv(rot=63) and b"rotated width" in rope_kv(rot=80)
    assert b"row stride" in rope_kv(ld=100)
    assert b"cache arguments missing" in rope_kv(write_kv=1)
    att = build.load("attention", (("HEAD_DIM", 64),))
    att.dlgo_attention_decode.restype = ctypes.c_char_p

    def decode(head_dim=64, n_heads=32, n_kv=8, max_pages=4, used=4, variant=0, ldq=2048):
        return att.dlgo_attention_decode(null, ldq, null, 2048, null, i64(0), 2, n_heads, n_kv, head_dim, null, null, null, max_pages,
                                         used, null, i64(0), i64(0), 0, ctypes.c_float(0.125), null, null, 0, 0, 0, 0, variant,
                                         null, null)
    assert b"built for head size 64, got 128" in decode(head_dim=128)
    assert b"bad sizes" in decode(n_heads=30)
    assert b"bound on the pages" in decode(used=5)
    assert b"unknown variant" in decode(variant=7)
    assert b"row strides" in decode(ldq=100)
