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
    "lmh_decode_step_extra": ("DecodeStepExtra", "DecodeStepExtra"),
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


# ---------------------------------------------------------------------------------------------
# Static walk of the Julia glue (no Julia here to run it): every function Luminal applies to the arrays
# that to_device returned, on the interpreter and compiled-graph call paths, must have a HipArray method.
# ---------------------------------------------------------------------------------------------
# (what Luminal calls, reference file, line, text expected on that line, regex of the glue's method)
ARRAY_PROTOCOL = [
    ("to_device(inputs, device)", "src/Execution.jl", 621, "to_device(initial_inputs, device)",
     r"^function to_device\(data::AbstractArray\{T,N\}, ::HIPDevice\)"),
    ("length(data) in realize_view", "src/Execution.jl", 95, "length(data)", r"^Base\.length\(a::HipArray\)"),
    ("Base.reshape(data, dims...) in realize_view", "src/Execution.jl", 96, "Base.reshape(data,",
     r"^Base\.reshape\(a::HipArray, dims::Int\.\.\.\)"),
    ("Base.reshape(data, fill(1, n)...) for one-element data", "src/Execution.jl", 103, "Base.reshape(data, fill(1",
     r"^function Base\.reshape\(a::HipArray\{T\}, dims::NTuple\{N,Int\}\)"),
    ("realize_view on every interpreter input", "src/Execution.jl", 639, "realize_view(raw_data, st)", None),
    ("execute_op(op, input_values...)", "src/Execution.jl", 652, "execute_op(op, input_values...)",
     r"^function execute_op\(op::FlashAttentionOp, q::HipArray, k::HipArray, v::HipArray\)"),
    ("similar(q) in execute_op", "src/Execution.jl", 253, "similar(q)", r"^Base\.similar\(a::HipArray\{T,N\}\)"),
    ("execute_op!(out, op, q, k, v)", "src/Execution.jl", 565, "function execute_op!(out, op::FlashAttentionOp",
     r"^function execute_op!\(out::HipArray\{TO,4\}, op::FlashAttentionOp, q::HipArray\{T,4\}"),
    ("from_device(results[id])", "src/Execution.jl", 662, "from_device(results[id])",
     r"^function from_device\(a::HipArray\{T,N\}\)"),
    ("length(cg.results[k]) in a compiled call", "src/Compiler.jl", 86, "length(cg.results[k])",
     r"^Base\.length\(a::HipArray\)"),
    ("copyto!(cg.results[k], v)", "src/Compiler.jl", 89, "copyto!(cg.results[k], v)",
     r"^function Base\.copyto!\(dst::HipArray\{T,N\}, src::AbstractArray\)"),
    ("copyto!(results[id], to_device(...)) for constants", "src/Compiler.jl", 230, "copyto!(results[node_id], to_device(",
     r"^function Base\.copyto!\(dst::HipArray\{T\}, src::HipArray\{T\}\)"),
    ("execute_with_capture(device, run_graph, cg.cache)", "src/Compiler.jl", 98, "execute_with_capture(device, run_graph, cg.cache)",
     r"^function execute_with_capture\(::HIPDevice, f, cache::Dict\)"),
    ("realize_view(results[id], st) captured by the step closure", "src/Compiler.jl", 252, "realize_view(results[id], st)",
     r"step_args = \[realize_view\(results\[id\], st\) for \(id, _, st\) in node\.inputs\]"),
    ("execute_op!(target_buf, op, step_args...)", "src/Compiler.jl", 254, "execute_op!(target_buf, op, step_args...)",
     r"push!\(steps, \(results, device\) -> execute_op!\(target_buf, op, step_args\.\.\.\)\)"),
    ("CompiledGraph(steps, results, cache)", "src/Compiler.jl", 75, "struct CompiledGraph",
     r"return Luminal\.CompiledGraph\(steps, results, cache\)"),
    # every other op the interpreter dispatches (src/Execution.jl:216-250) meets HipArray arguments on a HIPDevice:
    # a fallback method generated for each op type of Luminal's, for each pattern of HipArray positions
    ("execute_op(op::Add, a, b) and the other untyped CPU methods", "src/Execution.jl", 216, "execute_op(op::Add, a, b)",
     r"^for T in subtypes\(Op\)$"),
    ("execute_op(op::MatMul, a, b)", "src/Execution.jl", 231, "execute_op(op::MatMul, a, b)",
     r"@eval execute_op\(op::\$T, \$\(sig\.\.\.\)\) = host_fallback\(op, \$\(names\.\.\.\)\)"),
    ("execute_op(op::Reshape, a)", "src/Execution.jl", 228, "execute_op(op::Reshape, a)",
     r"^function host_fallback\(op::Op, args\.\.\.\)"),
]
EXTRA_METHODS = [  # used by the glue's own executors on HipArray arguments
    r"^Base\.size\(a::HipArray\)", r"^Base\.size\(a::HipArray, i::Integer\)", r"^Base\.ndims\(::HipArray\{T,N\}\)",
    r"^Base\.eltype\(::HipArray\{T\}\)", r"^to_device\(data::HipArray, ::HIPDevice\)",
    r"^function compile_hip\(graph::Luminal\.Graph",
]
REFERENCE = "/root/reference"


def glue_text():
    return open(os.path.join(ROOT, "luminal.jl_amd", "julia", "LuminalHIP.jl")).read()


def test_glue_defines_every_array_method_the_reference_call_paths_use():
    text = glue_text()
    for what, ref_file, ref_line, ref_text, pattern in ARRAY_PROTOCOL:
        if pattern is not None:
            assert re.search(pattern, text, flags=re.M), "no HipArray method for: %s (%s:%d)" % (what, ref_file, ref_line)
    for pattern in EXTRA_METHODS:
        assert re.search(pattern, text, flags=re.M), pattern
    # where a checkout of the reference is at hand, the cited lines must say what this table says they do
    if os.path.isdir(REFERENCE):
        for what, ref_file, ref_line, ref_text, _ in ARRAY_PROTOCOL:
            lines = open(os.path.join(REFERENCE, ref_file)).read().split("\n")
            window = "\n".join(lines[max(ref_line - 3, 0):ref_line + 2])
            assert ref_text in window, "%s:%d does not contain %r" % (ref_file, ref_line, ref_text)


def test_glue_graph_nodes_have_builders_and_executors():
    # N1 / N2 / N4 on the Julia side: the rotary embedding and the cache append are graph nodes with an Op struct,
    # a builder that calls add_op!, an in-place executor and an allocating one; compile_hip knows all four ops
    text = glue_text()
    for op, builder in (("DecodeAttentionOp", "decode_attention"), ("RotaryEmbeddingOp", "rotary_embedding"),
                        ("KVAppendOp", "kv_cache_append"), ("RopeFlashAttentionOp", "rope_flash_attention"),
                        ("DecodeStepOp", "decode_step")):
        assert re.search(r"^struct %s <: Op$" % op, text, flags=re.M), op
        body = re.search(r"^function %s\(.*?^end$" % builder, text, flags=re.M | re.S)
        assert body and "add_op!(" in body.group(0) and op + "(" in body.group(0), builder
        assert re.search(r"^function execute_op!\(out::HipArray\{\w+,\d\}, op::%s," % op, text, flags=re.M), op
        assert re.search(r"^execute_op\(op::%s, " % op, text, flags=re.M), op
    assert re.search(r"^const DeviceOp = Union\{FlashAttentionOp,RopeFlashAttentionOp,DecodeAttentionOp,DecodeStepOp,RotaryEmbeddingOp,KVAppendOp\}$",
                     text, flags=re.M)
    exported = re.search(r"^export (.*?)\n\n", text, flags=re.M | re.S).group(1)
    for name in ("compile_hip", "HipArray", "HIPDevice", "rotary_embedding", "kv_cache_append", "decode_attention",
                 "cached_self_attention_core", "self_attention_core", "enable_capture!", "rope_flash_attention",
                 "prompt_self_attention_core!", "decode_step", "DecodeStepOp", "decode_step_supported"):
        assert name in re.split(r"[,\s]+", exported), name


def _strip_julia(text):
    """Julia source with comments and string contents blanked (interpolations included), newlines kept."""
    out, i, n = [], 0, len(text)
    while i < n:
        c = text[i]
        if text.startswith('"""', i):
            j = text.index('"""', i + 3)
            out.append("".join(ch if ch == "\n" else " " for ch in text[i:j + 3]))
            i = j + 3
        elif c == '"':
            j = i + 1
            depth = 0
            while j < n and not (text[j] == '"' and depth == 0):
                if text[j] == "\\":
                    j += 1
                elif text.startswith("$(", j):
                    depth += 1
                    j += 1
                elif text[j] == "(" and depth > 0:
                    depth += 1
                elif text[j] == ")" and depth > 0:
                    depth -= 1
                j += 1
            out.append(" " * (j + 1 - i))
            i = j + 1
        elif c == "#":
            j = text.find("\n", i)
            j = n if j < 0 else j
            out.append(" " * (j - i))
            i = j
        else:
            out.append(c)
            i += 1
    return "".join(out)


def test_glue_blocks_and_brackets_balance():
    # a syntax slip (a missing `end`, an unclosed bracket) would otherwise go unnoticed until someone runs Julia
    code = _strip_julia(glue_text())
    depth_brackets, blocks = [], []
    openers = {"function", "struct", "if", "for", "while", "try", "let", "begin", "module", "macro", "quote", "do"}
    for m in re.finditer(r"[A-Za-z_!][A-Za-z_0-9!]*|[\[\](){}]", code):
        tok = m.group(0)
        if tok in "([{":
            depth_brackets.append(tok)
        elif tok in ")]}":
            assert depth_brackets, "unmatched %s at offset %d" % (tok, m.start())
            assert {"(": ")", "[": "]", "{": "}"}[depth_brackets.pop()] == tok, "bracket mismatch at offset %d" % m.start()
        elif depth_brackets:
            continue  # comprehensions (`for`, `if`) and `end` as an index live inside brackets
        elif tok in openers:
            if tok == "struct" and blocks and blocks[-1] == "mutable":
                blocks[-1] = "struct"
            else:
                blocks.append(tok)
        elif tok == "mutable":
            blocks.append("mutable")
        elif tok == "end":
            assert blocks, "`end` without an open block at offset %d" % m.start()
            blocks.pop()
    assert not depth_brackets and not blocks, (depth_brackets, blocks)


def _split_top_level(s):
    parts, depth, cur = [], 0, []
    for ch in s:
        if ch in "([{":
            depth += 1
        elif ch in ")]}":
            depth -= 1
        if ch == "," and depth == 0:
            parts.append("".join(cur).strip())
            cur = []
        else:
            cur.append(ch)
    if "".join(cur).strip():
        parts.append("".join(cur).strip())
    return parts


def test_glue_ccalls_pass_as_many_arguments_as_the_header_declares():
    code = _strip_julia(glue_text())
    protos = {name: args for name, args in re.findall(r"\b(lmh_\w+)\s*\(([^)]*)\)\s*;", header_text())}
    seen, names = 0, set()
    for m in re.finditer(r"ccall\(", code):
        i, depth = m.end(), 1
        while depth:
            depth += {"(": 1, ")": -1}.get(code[i], 0)
            i += 1
        parts = _split_top_level(code[m.end():i - 1])
        name = re.match(r"\(:(lmh_\w+)", parts[0]).group(1)
        types = _split_top_level(parts[2].strip()[1:-1])
        values = parts[3:]
        assert len(types) == len(values), "ccall of %s: %d types, %d values" % (name, len(types), len(values))
        declared = [a for a in protos[name].split(",") if a.strip() and a.strip() != "void"]
        assert len(declared) == len(types), "ccall of %s: header declares %d parameters" % (name, len(declared))
        # ... of the same kinds, in the same order, and the same return type
        for decl, jl in zip(declared, types):
            assert jl.strip() in _julia_spellings(decl), "ccall of %s: header parameter %r passed as %s" % (name, decl.strip(), jl.strip())
        ret = re.search(r"([\w ]+?[ *]+)%s\s*\(" % name, header_text()).group(1)
        assert parts[1].strip() in _julia_spellings(ret + "x"), "ccall of %s returns %r in the header, %s in the glue" % (name, ret, parts[1])
        seen += 1
        names.add(name)
    assert seen >= 20
    assert {"lmh_flash_attn_fwd", "lmh_flash_attn_plan", "lmh_decode_attn", "lmh_decode_attn_static", "lmh_decode_step", "lmh_rope",
            "lmh_kv_append"} <= names


def _julia_spellings(c_decl):
    """The ccall type spellings that fit one C parameter declaration (`const lmh_attn_params *p`, `size_t bytes` ...)."""
    d = " ".join(c_decl.replace("*", " * ").split())
    m = re.match(r"(?:const )?(\w+)((?: \*)*) \w+$", d)
    assert m, c_decl
    base, stars = m.group(1), m.group(2).count("*")
    struct = {"lmh_attn_params": "AttnParams", "lmh_decode_params": "DecodeParams", "lmh_rope_params": "RopeParams",
              "lmh_kv_append_params": "KvAppendParams", "lmh_decode_step_extra": "DecodeStepExtra"}
    if base in struct:
        assert stars == 1
        return {"Ref{%s}" % struct[base]}
    if stars == 0:
        return {"int": {"Cint", "Int32"}, "int32_t": {"Int32", "Cint"}, "size_t": {"Csize_t"}, "float": {"Float32", "Cfloat"}}[base]
    if base == "void":
        return {"Ptr{Cvoid}"} if stars == 1 else {"Ref{Ptr{Cvoid}}", "Ptr{Ptr{Cvoid}}"}
    if base == "char":
        return {"Ptr{UInt8}", "Cstring"}
    if base == "float":
        return {"Ref{Float32}", "Ptr{Float32}"}
    raise AssertionError("no Julia spelling known for %r" % c_decl)


def test_glue_host_fallback_and_layer_builder():
    """The fallback downloads, calls Luminal's own CPU method and uploads; compile_hip gives nodes without a kernel a
    host step instead of refusing them, and such graphs cannot be recorded; self_attention keeps the reference layer's
    projections and reshapes (reference src/NN.jl:343-361, :383-386) around self_attention_core."""
    text = glue_text()
    body = re.search(r"^function host_fallback\(op::Op, args\.\.\.\).*?^end$", text, flags=re.M | re.S).group(0)
    assert "execute_op(op, map(host_value, args)...)" in body and "to_device(" in body and "cache_capturing()" in body
    assert re.search(r"^host_value\(x::HipArray\) = from_device\(x\)$", text, flags=re.M)
    # the generated methods skip the ops that have kernels and the glue's own op types
    loop = re.search(r"^for T in subtypes\(Op\)\n(.*?)^end$", text, flags=re.M | re.S).group(1)
    assert "is_device_op_type(T) || parentmodule(T) === @__MODULE__" in loop and "pattern in 1:(2^n - 1)" in loop
    comp = re.search(r"^function compile_hip\(.*?^end$", text, flags=re.M | re.S).group(0)
    assert "copyto!(target_buf, Array(execute_op(op, map(host_value, step_args)...)))" in comp
    assert "has no executor" not in comp and ":hip_host_steps" in comp
    cap = re.search(r"^function enable_capture!\(.*?^end$", text, flags=re.M | re.S).group(0)
    assert ":hip_host_steps" in cap and "error(" in cap
    layer = re.search(r"^function self_attention\(sa::Luminal\.NN\.SelfAttention, x::GraphTensor, prev_seq::Int;.*?^end$", text,
                      flags=re.M | re.S).group(0)
    for piece in ("sa.q_proj", "sa.k_proj", "sa.v_proj", "sa.o_proj", "Luminal.reshape(proj(x), [batch, seq, n, sa.head_dim])",
                  "[1, 3, 2, 4]", "self_attention_core(queries, keys, values; causal=true, prev_seq=prev_seq, rope_base=rope_base)",
                  "[batch, seq, hidden]"):
        assert piece in layer, piece
    wh = re.search(r"^function whisper_attention\(layer, x::GraphTensor;.*?^end$", text, flags=re.M | re.S).group(0)
    for piece in ("layer.q_proj, x", "layer.k_proj, keys_from", "layer.v_proj, values_from", "layer.o_proj(out)",
                  "[b, s, n_heads, head_dim]", "[1, 3, 2, 4]", "Luminal.flash_attention(", "causal=mask", "[batch, seq, hidden]"):
        assert piece in wh, piece
    if os.path.isdir(REFERENCE):
        w = open(os.path.join(REFERENCE, "src/Whisper.jl")).read()
        assert "Luminal.permute(Luminal.reshape(sa.q_proj(x) * scale, [batch, seq, HEADS, HEAD_DIM]), [1, 3, 2, 4])" in w
        assert "scale = (Float32(hidden) / Float32(HEADS)) ^ -0.25f0" in w
    if os.path.isdir(REFERENCE):  # the layer's own lines in the reference say the same
        nn = open(os.path.join(REFERENCE, "src/NN.jl")).read()
        assert "Luminal.reshape(sa.q_proj(x), [batch, seq, sa.n_heads, sa.head_dim])" in nn
        assert "Luminal.permute(queries, [1, 3, 2, 4])" in nn and "Luminal.reshape(out, [batch, seq, hidden])" in nn


def test_glue_device_cache_mirrors_the_reference_cache_holder():
    """HipKVCache keeps what KVCacheState keeps for self attention (reference src/Whisper.jl:519-540: max_seq, one (K, V)
    pair per layer, zero-filled (B, H, max_seq, D)) and its step functions hand the cores exactly the keywords they take."""
    text = glue_text()
    st = re.search(r"^mutable struct HipKVCache\{T\}\n(.*?)^end$", text, flags=re.M | re.S).group(1)
    for field in ("max_seq::Int", "self_cache::Vector{Tuple{HipArray{T,4},HipArray{T,4}}}", "kv_len_host::Vector{Int32}",
                  "pos::HipArray{Int32,1}", "kv_len::HipArray{Int32,1}"):
        assert field in st, field
    ctor = re.search(r"^function HipKVCache\{T\}\(.*?^end$", text, flags=re.M | re.S).group(0)
    assert ctor.count("zeros_hip(T, (batch, n_kv_heads, max_seq, head_dim))") == 2 and "for _ in 1:n_layers" in ctor
    for fn, core in (("decode_layer!", "cached_self_attention_core!"), ("prompt_layer!", "prompt_self_attention_core!")):
        body = re.search(r"^function %s\(.*?^end$" % re.escape(fn), text, flags=re.M | re.S).group(0)
        call = re.search(r"%s\((.*?)\)\nend" % re.escape(core), body, flags=re.S).group(1)
        sig = re.search(r"^function %s\((.*?)\) where" % re.escape(core), text, flags=re.M | re.S).group(1)
        positional, keywords = sig.split(";")
        assert len(_split_top_level(call.split(";")[0])) == len(_split_top_level(positional)), fn
        for kw in re.findall(r"(\w+)=", call.split(";")[1]):
            assert re.search(r"\b%s(::\w+)?=" % kw, keywords), (fn, kw)
    begin = re.search(r"^function begin_step!\(.*?^end$", text, flags=re.M | re.S).group(0)
    assert "copyto!(c.pos, c.kv_len_host)" in begin and "c.kv_len_host .+ Int32(n_new)" in begin and "error(" in begin
    if os.path.isdir(REFERENCE):
        wh = open(os.path.join(REFERENCE, "src/Whisper.jl")).read()
        assert "self_cache::Vector{Tuple{Array{Float32,4}, Array{Float32,4}}}" in wh and "cache.step_pos += 1" in wh
