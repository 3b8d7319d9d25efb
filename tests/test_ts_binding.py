"""The Deno binding (gguf-trainer_amd/ts/hip.ts) against the C header, mechanically: its Deno.dlopen table names exactly
the entry points include/ggufhip.h declares, with every parameter and result type the FFI type that C type needs; the
ctypes table of the Python mirror is held to the same header; and the backend class carries every method of the
reference's OpsBackend / RegionBackend interfaces and of the buffer surface the trainer and the optimizers call
(src/model/autograd.ts:103-164, src/backend/webgpu.ts:393-862, 1432-1510)."""
import ctypes as C
import importlib
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TS = os.path.join(ROOT, "gguf-trainer_amd", "ts", "hip.ts")
HDR = os.path.join(ROOT, "include", "ggufhip.h")

# C parameter type -> Deno FFI type. Handles passed by value are pointers; anything the library reads from or writes to
# host memory is a TypedArray ("buffer"); device addresses are 64-bit integers.
HANDLES = {"gt_ctx *", "gt_adamw *", "gt_muon *"}
SCALARS = {"int": "i32", "float": "f32", "double": "f64", "size_t": "usize", "int64_t": "i64", "gt_buf": "u64", "uint64_t": "u64"}


def header_prototypes():
    src = open(HDR).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    src = re.sub(r"//[^\n]*", "", src)
    out = {}
    for m in re.finditer(r"\b(int|const char \*)\s*(gt_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", src, flags=re.S):
        ret, name, params = m.group(1), m.group(2), m.group(3)
        ps = []
        for p in [x.strip() for x in re.sub(r"\s+", " ", params).split(",")]:
            if p == "void" or not p:
                continue
            m2 = re.match(r"^(.*?)([A-Za-z_][A-Za-z0-9_]*)$", p)          # type, then the parameter's name
            ctype = m2.group(1).strip()
            ctype = re.sub(r"\s*\*\s*", " *", ctype).replace("* *", "**").strip()
            ps.append(ctype)
        out[name] = (ret.strip(), ps)
    return out


def ffi_type(ctype: str) -> str:
    c = ctype.replace("const ", "").strip()
    if c in HANDLES:
        return "pointer"
    if c.endswith("*"):
        return "buffer"
    return SCALARS[c]


def ts_table():
    src = open(TS).read()
    consts = dict(re.findall(r'(\w+) = "(\w+)"', src[src.index("const u64"):src.index("const SYMBOLS")]))
    body = src[src.index("const SYMBOLS = {"):src.index("} as const;")]
    out = {}
    for m in re.finditer(r"(gt_[a-z0-9_]+):\s*\{\s*parameters:\s*\[([^\]]*)\],\s*result:\s*(\w+)\s*\}", body):
        name, params, res = m.groups()
        toks = [t.strip() for t in params.split(",") if t.strip()]
        out[name] = ([consts.get(t, t.strip('"')) for t in toks], consts.get(res, res))
    return out


def test_dlopen_table_matches_the_header_symbol_for_symbol_and_type_for_type():
    protos, table = header_prototypes(), ts_table()
    assert len(protos) >= 60
    assert sorted(table) == sorted(protos), (sorted(set(protos) - set(table)), sorted(set(table) - set(protos)))
    for name, (ret, params) in protos.items():
        want = [ffi_type(p) for p in params]
        got, gres = table[name]
        assert got == want, f"{name}: hip.ts has {got}, the header needs {want} ({params})"
        assert gres == ("pointer" if ret.endswith("*") else "i32"), name


def test_ctypes_table_matches_the_header_type_for_type():
    lib = importlib.import_module("gguf-trainer_amd.lib")
    protos = header_prototypes()
    size = {"i32": 4, "f32": 4, "f64": 8, "i64": 8, "u64": 8, "usize": C.sizeof(C.c_size_t)}
    for name, (ret, params) in protos.items():
        fn = getattr(lib.lib, name)
        assert len(fn.argtypes) == len(params), name
        for ct, p in zip(fn.argtypes, params):
            want = ffi_type(p)
            if want in ("pointer", "buffer"):
                assert ct in (C.c_void_p, C.c_char_p) or issubclass(ct, C._Pointer), (name, p, ct)
            else:
                assert not issubclass(ct, C._Pointer) and C.sizeof(ct) == size[want], (name, p, ct)
                is_float = ct in (C.c_float, C.c_double)
                assert is_float == (want in ("f32", "f64")), (name, p, ct)


def test_backend_class_has_the_reference_surface():
    src = open(TS).read()
    cls = src[src.index("export class HipBackend implements OpsBackend, RegionBackend"):src.index("// ---- optimizers")]
    ops = ["linear", "add", "mul", "silu", "gelu", "scale", "rmsNorm", "rmsNormHeads", "embedding", "rope", "attention",
           "crossEntropy", "fusedCrossEntropy", "softCrossEntropy"]                         # autograd.ts:103-151
    region = ["beginRegion", "endRegion", "seedGradFrom"]                                   # autograd.ts:160-164
    surface = ["install", "uninstall", "uploadParams", "sync", "reclaimStepTransients", "seedGradFromHost", "buffersFor",
               "keepGradOnDevice", "createStateBuffer", "writeStateBuffer", "readStateBuffer", "residentBytes",
               "regionCount", "startProfile", "stopProfile", "destroy"]                     # webgpu.ts:393-862, 1432-1510
    for m in ops + region + surface:
        assert re.search(rf"^\s+(async\s+)?{m}\(", cls, flags=re.M), f"HipBackend.{m} is missing"
    for field in ("attnFlashMinT", "lastSyncReadbackBytes", "gradClearsIssued", "adapterName"):
        assert re.search(rf"^\s+(readonly\s+)?{field}\b", cls, flags=re.M), field
    for name, methods in (("AdamWHip", ["setLrScale", "zeroGrad", "recordStep", "syncWeightsToHost", "exportState", "importState"]),
                          ("MuonHip", ["setLrScale", "zeroGrad", "recordStep", "syncWeightsToHost", "exportState", "importState"])):
        body = src[src.index(f"export class {name}"):]
        body = body[:body.index("\n}\n") + 3]
        for m in methods:
            assert re.search(rf"^\s+(async\s+)?{m}\(", body, flags=re.M), f"{name}.{m} is missing"
    for fn in ("initHip", "requireHip", "newtonSchulzHip"):
        assert f"export async function {fn}(" in src
    # every symbol the code calls is in the table, and brackets balance (a cheap stand-in for a parser)
    called = set(re.findall(r"\.(gt_[a-z0-9_]+)\b", src))
    assert called <= set(ts_table()), called - set(ts_table())
    for a, b in ("()", "[]", "{}"):
        stripped = re.sub(r"//[^\n]*|`[^`]*`|\"[^\"\n]*\"", "", src)
        assert stripped.count(a) == stripped.count(b), (a, stripped.count(a), stripped.count(b))


def _calls(src: str):
    """(name, [argument texts]) of every direct call `….gt_name(…)` in the TypeScript source, arguments split at top-level commas."""
    src = re.sub(r"//[^\n]*", "", src)
    out = []
    for m in re.finditer(r"\.(gt_[a-z0-9_]+)\(", src):
        i, depth, args, cur, quote = m.end(), 1, [], "", None
        while depth:
            ch = src[i]
            if quote:
                cur += ch
                if ch == quote and src[i - 1] != "\\":
                    quote = None
            elif ch in "\"'`":
                quote = ch
                cur += ch
            elif ch in "([{":
                depth += 1
                cur += ch
            elif ch in ")]}":
                depth -= 1
                if depth:
                    cur += ch
            elif ch == "," and depth == 1:
                args.append(cur.strip())
                cur = ""
            else:
                cur += ch
            i += 1
        if cur.strip():
            args.append(cur.strip())
        out.append((m.group(1), args))
    return out


def test_every_call_in_the_binding_passes_what_the_header_declares():
    """Deno.dlopen checks nothing until a call is made, and the binding cannot be run here: every direct call of a library
    symbol in hip.ts must pass exactly as many arguments as the header's prototype has parameters, no BigInt where the
    parameter is a 32-bit integer or a float, and no float literal or array where it is an integer."""
    protos = header_prototypes()
    calls = _calls(open(TS).read())
    assert len(calls) >= 70
    seen = set()
    for name, args in calls:
        ret, params = protos[name]
        assert len(args) == len(params), f"{name}: called with {len(args)} arguments {args}, the header declares {len(params)}"
        seen.add(name)
        for a, p in zip(args, params):
            want = ffi_type(p)
            if want in ("i32", "f32", "f64"):
                assert not re.fullmatch(r"\d+n", a) and not a.startswith("BigInt("), f"{name}: BigInt {a!r} for {p}"
            if want in ("i32", "i64", "u64", "usize"):
                assert not re.fullmatch(r"\d+\.\d+", a) and not a.startswith("["), f"{name}: {a!r} for {p}"
            if want == "pointer":
                assert re.fullmatch(r"null|(\w+\.)*(ctx|context|handle)", a), f"{name}: {a!r} where the handle {p} goes"
    # the binding exercises the whole path: every op's forward and backward entry point, the optimizers, the buffer calls
    for must in ("gt_gemm", "gt_rmsnorm_fwd", "gt_rmsnorm_bwd", "gt_rope", "gt_attn_fwd_scores", "gt_attn_bwd_scores", "gt_ce_fwd", "gt_ce_bwd",
                 "gt_embedding_fwd", "gt_embedding_bwd", "gt_glu_fwd", "gt_glu_bwd", "gt_adamw_step", "gt_muon_step", "gt_sync", "gt_h2d", "gt_d2h"):
        assert must in seen, must
