"""The three descriptions of the C ABI's parameter structs — include/luminal_hip.h, the ctypes mirror in
binding.py and the Julia glue (shipped as source; no Julia here to run it) — must list the same fields, with the
same kinds, in the same order, and the glue may only call symbols the header declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
STRUCTS = {  # header name -> (ctypes class, Julia struct)
    "lmh_attn_params": ("AttnParams", "AttnParams"),
    "lmh_decode_params": ("DecodeParams", "DecodeParams"),
    "lmh_rope_params": ("RopeParams", "RopeParams"),
    "lmh_kv_append_params": ("KvAppendParams", "KvAppendParams"),
}


def header_text():
    text = open(os.path.join(ROOT, "include", "luminal_hip.h")).read()
    return re.sub(r"/\*.*?\*/", "", text, flags=re.S)


def header_structs():
    out = {}
    for body, name in re.findall(r"typedef struct \w+ \{(.*?)\}\s*(\w+);", header_text(), flags=re.S):
        fields = []
        for decl in body.split(";"):
            decl = " ".join(decl.split())
            if not decl:
                continue
            m = re.match(r"(const )?(void|int32_t|int64_t|float|size_t) ?(\*)? ?(.*)", decl)
            assert m, decl
            base, star, names = m.group(2), m.group(3), m.group(4)
            for item in names.split(","):
                item = item.strip()
                am = re.match(r"(\w+)\[(\d+)\]", item)
                nm, count = (am.group(1), int(am.group(2))) if am else (item, 1)
                kind = "ptr" if star else {"int32_t": "i32", "int64_t": "i64", "float": "f32", "size_t": "size"}[base]
                fields.append((nm, kind, count))
        out[name] = fields
    return out


def ctypes_fields(cls):
    kinds = {ctypes.c_void_p: "ptr", ctypes.c_int32: "i32", ctypes.c_int64: "i64", ctypes.c_float: "f32",
             ctypes.c_size_t: "size"}
    out = []
    for name, ty in cls._fields_:
        if hasattr(ty, "_length_"):
            out.append((name, kinds[ty._type_], ty._length_))
        else:
            out.append((name, kinds[ty], 1))
    return out


def julia_structs():
    text = open(os.path.join(ROOT, "luminal.jl_amd", "julia", "LuminalHIP.jl")).read()
    out = {}
    for name, body in re.findall(r"^struct (\w+)\n(.*?)^end", text, flags=re.S | re.M):
        fields = []
        for decl in re.split(r"[;\n]", body):
            decl = decl.strip()
            if not decl or decl.startswith("#"):
                continue
            nm, ty = [x.strip() for x in decl.split("::")]
            tm = re.match(r"NTuple\{(\d+),Int64\}", ty)
            if tm:
                fields.append((nm, "i64", int(tm.group(1))))
            else:
                kind = {"Int32": "i32", "Float32": "f32", "Csize_t": "size"}.get(ty) or ("ptr" if ty.startswith("Ptr{") else None)
                assert kind, (name, decl)
                fields.append((nm, kind, 1))
        out[name] = fields
    return text, out


def test_ctypes_mirror_matches_the_header(lm):
    hs = header_structs()
    for cname, (pyname, _) in STRUCTS.items():
        assert ctypes_fields(getattr(lm.binding, pyname)) == hs[cname], cname


def test_julia_glue_matches_the_header():
    hs = header_structs()
    text, js = julia_structs()
    for cname, (_, jname) in STRUCTS.items():
        assert js[jname] == hs[cname], cname
    declared = set(re.findall(r"\b(lmh_\w+)\s*\(", header_text()))
    called = set(re.findall(r"\(:(lmh_\w+),", text))
    assert called and called <= declared, called - declared
    # the constants the glue repeats
    for name, value in re.findall(r"#define (LMH_(?:F32|F16|BF16|HEADMAP_INTERLEAVED|HEADMAP_BLOCKED)) (\d+)", header_text()):
        m = re.search(r"\b%s\b[^\n]*" % name.replace("LMH_HEADMAP", "HEADMAP"), text)
        assert m, name
    codes = re.search(r"const LMH_F32, LMH_F16, LMH_BF16 = Int32\((\d)\), Int32\((\d)\), Int32\((\d)\)", text)
    want = dict(re.findall(r"#define (LMH_(?:F32|F16|BF16)) (\d+)", header_text()))
    assert codes and list(codes.groups()) == [want["LMH_F32"], want["LMH_F16"], want["LMH_BF16"]]
