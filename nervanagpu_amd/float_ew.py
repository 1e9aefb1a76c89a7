"""
Fused elementwise / reduction / broadcast kernels, generated at run time.

Host-side counterpart of the reference's compound-kernel generator
(nervanagpu/float_ew.py:540-1322): a postfix expression stack is turned into
ONE kernel that keeps every intermediate in fp32 registers, performs all
reductions of the expression along one axis, and rounds once on the final
store (nearest, or stochastic for fp16/fp32 outputs).  Same operator
vocabulary (op table float_ew.py:464-533), same broadcasting rules
(:1156-1218), same de-duplication of repeated reductions (:614-647), same
argmax/argmin tie rule (lower index wins, :519-532).

What is different is the kernel shape, chosen for CDNA4:
  * the source is HIP, compiled with hiprtc for gfx950 and cached per
    expression signature;
  * a workgroup owns one row (the reduced axis) and lanes own 16-byte vectors of
    consecutive elements whenever the operands are contiguous and aligned;
  * when the row fits in registers (<= 32 values per lane) every operand is read
    from memory exactly once and all reduction stages run on the cached
    registers, so e.g. batch normalisation moves 1 read + 1 write per element
    instead of 3 reads + 1 write;
  * reductions are 64-lane butterfly shuffles, LDS is only used to combine
    wavefronts;
  * plain contiguous expressions (no reduction / broadcast / transpose / take)
    run as one flat grid-stride kernel instead of one workgroup per 256 elements;
  * stochastic rounding draws from a counter-based stream keyed on
    (seed, launch counter, logical element index), so results are reproducible.
"""
import ctypes
from ctypes import c_float, c_int, c_long, c_uint, c_void_p

import numpy as np

from . import _lib

# op name -> (operand count, C expression); {0},{1} are the operands in source order.
# The reference builds its kernels with --use_fast_math (nervanagpu/float_ew.py:1030):
# division and square root are the hardware approximations (about 1 ulp), not
# the correctly rounded sequences.
_float_ops = {
    "assign":  (2, None),
    "add":     (2, "({0} + {1})"),
    "sub":     (2, "({0} - {1})"),
    "mul":     (2, "({0} * {1})"),
    "div":     (2, "({0} * __builtin_amdgcn_rcpf({1}))"),
    "eq":      (2, "(({0} == {1}) ? 1.0f : 0.0f)"),
    "ne":      (2, "(({0} != {1}) ? 1.0f : 0.0f)"),
    "lt":      (2, "(({0} <  {1}) ? 1.0f : 0.0f)"),
    "le":      (2, "(({0} <= {1}) ? 1.0f : 0.0f)"),
    "gt":      (2, "(({0} >  {1}) ? 1.0f : 0.0f)"),
    "ge":      (2, "(({0} >= {1}) ? 1.0f : 0.0f)"),
    "minimum": (2, "fminf({0}, {1})"),
    "maximum": (2, "fmaxf({0}, {1})"),
    "pow":     (2, "powf({0}, {1})"),
    "finite":  (1, "(isfinite({0}) ? 1.0f : 0.0f)"),
    "neg":     (1, "(-{0})"),
    "abs":     (1, "fabsf({0})"),
    "sgn":     (1, "copysignf(1.0f, {0})"),
    "sqrt":    (1, "__builtin_amdgcn_sqrtf({0})"),
    "sqr":     (1, "({0} * {0})"),
    "exp":     (1, "expf({0})"),
    "log":     (1, "logf({0})"),
    "exp2":    (1, "exp2f({0})"),
    "log2":    (1, "log2f({0})"),
    "sig":     (1, "__builtin_amdgcn_rcpf(1.0f + expf(-{0}))"),
    "sig2":    (1, "__builtin_amdgcn_rcpf(1.0f + exp2f(-{0}))"),
    "tanh":    (1, "tanhf({0})"),
    "tanh2":   (1, "((exp2f(2.0f * {0}) - 1.0f) * __builtin_amdgcn_rcpf(exp2f(2.0f * {0}) + 1.0f))"),
    "rand":    (0, None),
    "onehot":  (0, None),
}

_reduction_ops = ("sum", "max", "min", "argmax", "argmin")

_ew_types = {
    "f4": ("float", None),
    "f2": ("_Float16", None),
    "i4": ("int", (-2147483648.0, 2147483520.0)),
    "u4": ("unsigned int", (0.0, 4294967040.0)),
    "i2": ("short", (-32768.0, 32767.0)),
    "u2": ("unsigned short", (0.0, 65535.0)),
    "i1": ("signed char", (-128.0, 127.0)),
    "u1": ("unsigned char", (0.0, 255.0)),
}

MAX_CACHED_PER_LANE = 32     # fp32 registers per operand kept resident per lane
MAX_THREADS = 1024
FLAT_UNROLL = 4              # independent vectors per lane per pass of the flat kernel


def _contiguous_strides(shape):
    if not shape:
        return ()
    strides = [1]
    for s in shape[:0:-1]:
        strides.append(strides[-1] * s)
    return tuple(strides[::-1])


_fast_dims_cache = {}


def _get_fast_ew_dims(size):
    """(shape, strides) of the 2-D view under which the reference runs a flat
    contiguous tensor (nervanagpu/float_ew.py:1037-1055): rows of the widest
    length that divides `size`, tried first among the multiples of 32 from 256
    down, then among all lengths from 255 down (1 always divides).  This
    generator runs flat expressions as a single row; the function remains for
    callers that shape their own views the reference's way."""
    if size not in _fast_dims_cache:
        candidates = list(range(256, 0, -32)) + list(range(255, 0, -1))
        width = next(w for w in candidates if size % w == 0)
        shape = (size // width, width)
        _fast_dims_cache[size] = (shape, _contiguous_strides(shape))
    return _fast_dims_cache[size]


# ---------------------------------------------------------------------------
# expression tree
# ---------------------------------------------------------------------------

class _Node(object):
    """kind: 'tensor' | 'const' | 'op' | 'red'.  key: structural identity used
    to merge repeated sub-expressions (and in particular repeated reductions)."""
    __slots__ = ("kind", "name", "args", "arg_id", "key", "level", "scalar", "extra", "op_id")

    def __init__(self, kind, name=None, args=(), arg_id=None, extra=None, op_id=None):
        self.kind, self.name, self.args, self.arg_id = kind, name, tuple(args), arg_id
        self.extra, self.op_id = extra, op_id
        if kind == "tensor":
            self.key = ("t", arg_id)
            self.level, self.scalar = 0, False
        elif kind == "const":
            self.key = ("c", arg_id)
            self.level, self.scalar = 0, True
        elif kind == "red":
            self.key = ("r", name, args[0].key)
            self.level, self.scalar = args[0].level + 1, True
        else:
            if name in ("rand", "onehot"):
                self.key = ("o", name, op_id)
                self.level, self.scalar = 0, False
            else:
                self.key = ("o", name) + tuple(a.key for a in args)
                self.level = max([a.level for a in args] + [0])
                self.scalar = all(a.scalar for a in args)


def _build_tree(type_args):
    """postfix description -> tree; returns (out_spec, root expression, assign spec)"""
    stack = []
    for arg in type_args:
        kind = arg[0]
        if kind == "tensor":
            stack.append(_Node("tensor", arg_id=arg[1]))
        elif kind == "const":
            stack.append(_Node("const", arg_id=arg[1]))
        elif kind == "assign":
            value = stack.pop()
            out = stack.pop()
            assert not stack, "malformed expression stack"
            return out, value, arg
        elif kind in _reduction_ops:
            stack.append(_Node("red", kind, [stack.pop()], op_id=arg[1]))
        else:
            nops = _float_ops[kind][0]
            operands = [stack.pop() for _ in range(nops)][::-1]
            stack.append(_Node("op", kind, operands, extra=arg[2:], op_id=arg[1]))
    raise ValueError("expression does not end in an assignment")


def _collect_reductions(node, found):
    for a in node.args:
        _collect_reductions(a, found)
    if node.kind == "red" and node.key not in found:
        found[node.key] = node
    return found


class _Emitter(object):
    """Turns a tree into HIP source for one kernel specialisation."""

    def __init__(self, spec):
        self.spec = spec
        self.lines = []
        self.names = {}          # key -> variable holding a row-scalar value
        self.counter = 0

    def fresh(self, prefix="r"):
        self.counter += 1
        return "%s%d" % (prefix, self.counter)

    # -- operand access ------------------------------------------------------
    def load_expr(self, tid, v):
        """float value of element v of the current vector of tensor tid"""
        return "x%d_%s[%s]" % (tid, self.cur_item, v)

    def emit_scalar(self, node, out):
        """value of a row-scalar node, emitted once at workgroup scope"""
        if node.key in self.names:
            return self.names[node.key]
        if node.kind == "const":
            name = "c%d" % node.arg_id
        elif node.kind == "red":
            raise AssertionError("reduction used before its stage")
        else:
            ops = [self.emit_scalar(a, out) for a in node.args]
            name = self.fresh("s")
            out.append("    const float %s = %s;" % (name, _float_ops[node.name][1].format(*ops)))
        self.names[node.key] = name
        return name

    def emit_elem(self, node, out, local, item, v):
        """value of a node for element (item, v) of the row, emitted in a loop body"""
        if node.scalar:
            return self.names[node.key] if node.key in self.names else self._late_scalar(node)
        if node.key in local:
            return local[node.key]
        if node.kind == "tensor":
            name = self.spec.tensor_value(node.arg_id, item, v)
        elif node.name == "rand":
            name = self.fresh("e")
            out.append("            const float %s = ng_frand(rng_seed, rng_stream + %du, rng_idx + %s);"
                       % (name, 0x1000193 * (node.op_id + 1) & 0xFFFFFFFF, v))
        elif node.name == "onehot":
            name = self.fresh("e")
            hot_axis, slot = node.extra
            test = "(col + %s)" % v if hot_axis == 1 else "row"
            idx = "oh%d_v" % slot if hot_axis == 0 else "oh%d_row" % slot
            if hot_axis == 0:
                out.append("            const float %s = (oh%d[col + %s] == %s) ? 1.0f : 0.0f;" % (name, slot, v, "row"))
            else:
                out.append("            const float %s = (%s == %s) ? 1.0f : 0.0f;" % (name, idx, test))
        else:
            ops = [self.emit_elem(a, out, local, item, v) for a in node.args]
            name = self.fresh("e")
            out.append("            const float %s = %s;" % (name, _float_ops[node.name][1].format(*ops)))
        local[node.key] = name
        return name

    def _late_scalar(self, node):
        raise AssertionError("row-scalar %r was not materialised before use" % (node.key,))

    def prepare_scalars(self, node, out, max_level):
        """emit every row-scalar subtree of `node` whose reductions are done"""
        if node.scalar:
            if node.kind == "red":
                assert node.key in self.names
                return
            if node.level <= max_level:
                self.emit_scalar_tree(node, out)
            return
        for a in node.args:
            self.prepare_scalars(a, out, max_level)

    def emit_scalar_tree(self, node, out):
        if node.key in self.names:
            return self.names[node.key]
        if node.kind == "red":
            raise AssertionError("reduction not computed yet")
        return self.emit_scalar(node, out)


class KernelSpec(object):
    """Everything that selects a generated kernel (hashable via .key)."""

    def __init__(self, type_args, tensors, mode, vec, threads, items, n_onehot, rng_pair=False):
        # tensors: list of (arg_id, dtype_code, access, take_axis, is_out)
        #   access: 'vec' contiguous+aligned along the row, 'strided', 'row' (one value per row)
        self.type_args = tuple(type_args)
        self.tensors = tuple(tensors)
        self.mode = mode              # 'flat' | 'row'
        self.vec = vec
        self.threads = threads
        self.items = items            # >0: row cached in registers with this many vectors per lane; 0: streaming
        self.n_onehot = n_onehot
        # rng_pair: vector stores start at an even random-stream index with unit
        # stride, so fp16 stochastic stores can share one draw per element pair
        self.rng_pair = bool(rng_pair)
        self.key = (self.type_args, self.tensors, mode, vec, threads, items, n_onehot, self.rng_pair)
        self._tensor_by_id = dict((t[0], t) for t in tensors)

    def tensor_value(self, arg_id, item, v):
        t = self._tensor_by_id[arg_id]
        if t[2] == "row":
            return "x%d_row" % arg_id
        return "x%d_%s[%s]" % (arg_id, item, v)


def _ctype(code):
    return _ew_types[code][0]


def _gen_load(spec, t, item, base_col, out, indent, bound="n"):
    """code that fills float x<id>_<item>[VEC] for the vector starting at column base_col"""
    arg_id, code, access, take_axis, _ = t
    V = spec.vec
    ct = _ctype(code)
    pad = " " * indent
    if access == "row":
        return
    out.append("%sfloat x%d_%s[%d];" % (pad, arg_id, item, V))
    if access == "vec" and V > 1:
        out.append("%s{ typedef %s vt_ __attribute__((ext_vector_type(%d)));" % (pad, ct, V))
        out.append("%s  const vt_ raw_ = *reinterpret_cast<const vt_*>(p%d + (long)(%s));" % (pad, arg_id, base_col))
        out.append("%s  _Pragma(\"unroll\") for (int v = 0; v < %d; v++) x%d_%s[v] = (float)raw_[v]; }" % (pad, V, arg_id, item))
    else:
        if take_axis == 2:
            idx = "(long)take%d[%s + v]" % (arg_id, base_col)
        else:
            idx = "(long)(%s + v) * cs%d" % (base_col, arg_id)
        out.append("%s_Pragma(\"unroll\") for (int v = 0; v < %d; v++)" % (pad, V))
        out.append("%s    x%d_%s[v] = (%s + v < %s) ? (float)p%d[%s] : 0.0f;" % (pad, arg_id, item, base_col, bound, arg_id, idx))


def _gen_round(code, value, rounding, idx, rword=None):
    """expression of storage type for fp32 `value`; `rword` overrides the
    random word of an fp16 stochastic store (shared pair draws)"""
    ct, rng = _ew_types[code]
    if code == "f4":
        if rounding:
            return "ng_sr_f32(%s, sr_bits, ng_rand32(rng_seed, rng_stream, %s))" % (value, idx)
        return value
    if code == "f2":
        if rounding:
            if rword is None:
                rword = "ng_rand_sr16(rng_seed, rng_stream, %s)" % idx
            return "__builtin_bit_cast(_Float16, ng_sr_f16(%s, sr_bits, %s))" % (value, rword)
        return "(_Float16)(%s)" % value
    return "(%s)ng_rint_sat(%s, %rf, %rf)" % (ct, value, rng[0], rng[1])


def generate_source(spec, name="ew_kernel"):
    """HIP source of the kernel described by `spec`.
    Returns (source, arg_order) where arg_order lists the launch arguments:
    ('ptr', id) ('rs', id) ('cs', id) ('take', id) ('const', id) ('onehot', slot)
    ('n',) ('n_out',) ('rows',) ('sr_bits',) ('rng_seed',) ('rng_stream',) ('rng_rm',) ('rng_cm',)"""
    out_node, root, assign = _build_tree(spec.type_args)
    rounding = bool(assign[2])
    reds = list(_collect_reductions(root, {}).values())
    reds.sort(key=lambda r: r.level)
    levels = sorted(set(r.level for r in reds))
    V, T, ITEMS = spec.vec, spec.threads, spec.items
    flat = spec.mode == "flat"
    out_t = [t for t in spec.tensors if t[4]][0]
    in_ts = [t for t in spec.tensors if not t[4]]
    red_out = root.scalar and not flat   # one value per row: lane 0 stores it

    args, decl = [], []
    for t in spec.tensors:
        arg_id, code, access, take_axis, is_out = t
        const = "" if is_out else "const "
        decl.append("%s%s* __restrict__ p%d" % (const, _ctype(code), arg_id))
        args.append(("ptr", arg_id))
        if not flat:
            decl.append("int rs%d" % arg_id); args.append(("rs", arg_id))
            decl.append("int cs%d" % arg_id); args.append(("cs", arg_id))
        if take_axis:
            decl.append("const int* __restrict__ take%d" % arg_id); args.append(("take", arg_id))
    consts = sorted(set(a[1] for a in spec.type_args if a[0] == "const"))
    for c in consts:
        decl.append("float c%d" % c); args.append(("const", c))
    for s in range(spec.n_onehot):
        decl.append("const int* __restrict__ oh%d" % s); args.append(("onehot", s))
    decl.append("int n"); args.append(("n",))
    decl.append("int n_out"); args.append(("n_out",))
    decl.append("long rows"); args.append(("rows",))
    decl += ["unsigned sr_bits", "unsigned rng_seed", "unsigned rng_stream", "unsigned rng_rm", "unsigned rng_cm"]
    args += [("sr_bits",), ("rng_seed",), ("rng_stream",), ("rng_rm",), ("rng_cm",)]

    em = _Emitter(spec)
    L = []
    L.append(_lib.common_header_text())
    L.append("#define THREADS %d" % T)
    L.append("#define VEC %d" % V)
    L.append("extern \"C\" __global__ __launch_bounds__(THREADS) void %s(\n    %s)\n{" % (name, ",\n    ".join(decl)))
    L.append("    const int tid = threadIdx.x;")

    def pair_words(o, pad, code):
        """shared draws for a vector of fp16 stochastic stores"""
        if not (spec.rng_pair and rounding and code == "f2"):
            return [None] * V
        for k in range(V // 2):
            o.append("%sconst unsigned rh%d_ = ng_rand32(rng_seed, rng_stream, (rng_idx >> 1) + %du);" % (pad, k, k))
        return ["rh%d_" % (v // 2) if v % 2 == 0 else "(rh%d_ << 16)" % (v // 2) for v in range(V)]

    def rounded_vector(o, pad, code, vals, rwords, idx_of):
        """statements that fill the vector o_ with the rounded values"""
        paired = rwords[0] is not None and V % 2 == 0
        if paired:
            # all 10 mantissa bits kept: pairs share a draw and a packed convert
            o.append("%sif (sr_bits == 10u) {" % pad)
            if V == 2:
                o.append("%s  o_ = __builtin_bit_cast(vt_, ng_sr10_f16x2(%s, %s, rh0_));" % (pad, vals[0], vals[1]))
            else:
                o.append("%s  typedef unsigned qt_ __attribute__((ext_vector_type(%d))); qt_ q_;" % (pad, V // 2))
                for k in range(V // 2):
                    o.append("%s  q_[%d] = ng_sr10_f16x2(%s, %s, rh%d_);" % (pad, k, vals[2 * k], vals[2 * k + 1], k))
                o.append("%s  o_ = __builtin_bit_cast(vt_, q_);" % pad)
            o.append("%s} else {" % pad)
        for v in range(V):
            o.append("%so_[%d] = %s;" % (pad, v, _gen_round(code, vals[v], rounding, idx_of(v), rwords[v])))
        if paired:
            o.append("%s}" % pad)

    def store_code(item, base_col, vals, indent):
        pad = " " * indent
        arg_id, code, access, take_axis, _ = out_t
        ct = _ctype(code)
        o = []
        if access == "vec" and V > 1:
            o.append("%s{ typedef %s vt_ __attribute__((ext_vector_type(%d))); vt_ o_;" % (pad, ct, V))
            rwords = pair_words(o, pad + "  ", code)
            rounded_vector(o, pad + "  ", code, vals, rwords,
                           lambda v: "rng_idx + %du" % v if not rng_strided else "rng_idx + %du * rng_cm" % v)
            o.append("%s  *reinterpret_cast<vt_*>(p%d + (long)(%s)) = o_; }" % (pad, arg_id, base_col))
        else:
            for v in range(V):
                if take_axis == 2:
                    idx = "(long)take%d[%s + %d]" % (arg_id, base_col, v)
                else:
                    idx = "(long)(%s + %d) * cs%d" % (base_col, v, arg_id)
                rid = "rng_idx + %du" % v if not rng_strided else "rng_idx + %du * rng_cm" % v
                o.append("%sif (active && %s + %d < n_out) p%d[%s] = %s;" % (pad, base_col, v, arg_id, idx, _gen_round(code, vals[v], rounding, rid)))
        return o

    uses_rand = any(a[0] == "rand" for a in spec.type_args)
    need_idx = rounding or uses_rand

    if flat:
        rng_strided = False
        # each workgroup walks chunks of FLAT_UNROLL * THREADS vectors; inside a
        # full chunk the per-vector bodies are independent, so their loads issue
        # back to back before the first use
        L.append("    const long nvec = rows;   // number of VEC-wide vectors")
        L.append("    auto vec_body = [&](const long g) {")
        L.append("        const long col = g * VEC;")
        L.append("        const unsigned rng_idx = (unsigned)col;")
        body = []
        for t in in_ts:
            arg_id, code, access, _, _ = t
            ct = _ctype(code)
            body.append("        float x%d_i[%d];" % (arg_id, V))
            if V > 1:
                body.append("        { typedef %s vt_ __attribute__((ext_vector_type(%d)));" % (ct, V))
                body.append("          const vt_ raw_ = *reinterpret_cast<const vt_*>(p%d + col);" % arg_id)
                body.append("          _Pragma(\"unroll\") for (int v = 0; v < %d; v++) x%d_i[v] = (float)raw_[v]; }" % (V, arg_id))
            else:
                body.append("        x%d_i[0] = (float)p%d[col];" % (arg_id, arg_id))
        for c in consts:
            em.names[("c", c)] = "c%d" % c
        vals = []
        for v in range(V):
            local = {}
            blk = []
            em.prepare_scalars(root, blk, 0)
            vals.append(em.emit_elem(root, blk, local, "i", str(v)) if not root.scalar else em.emit_scalar_tree(root, blk))
            body += ["    " + b[4:] if b.startswith("            ") else b for b in blk]
        L += body
        arg_id, code, _, _, _ = out_t
        ct = _ctype(code)
        if V > 1:
            L.append("        { typedef %s vt_ __attribute__((ext_vector_type(%d))); vt_ o_;" % (ct, V))
            rwords = pair_words(L, "          ", code)
            rounded_vector(L, "          ", code, vals, rwords, lambda v: "rng_idx + %du" % v)
            L.append("          *reinterpret_cast<vt_*>(p%d + col) = o_; }" % arg_id)
        else:
            L.append("        p%d[col] = %s;" % (arg_id, _gen_round(code, vals[0], rounding, "rng_idx")))
        L.append("    };")
        L.append("    const long chunk = (long)THREADS * %d;" % FLAT_UNROLL)
        L.append("    for (long base = (long)blockIdx.x * chunk; base < nvec; base += (long)gridDim.x * chunk) {")
        L.append("        if (base + chunk <= nvec) {")
        L.append("            _Pragma(\"unroll\") for (int u = 0; u < %d; u++) vec_body(base + (long)u * THREADS + tid);" % FLAT_UNROLL)
        L.append("        } else {")
        L.append("            for (long g = base + tid; g < nvec; g += THREADS) vec_body(g);")
        L.append("        }")
        L.append("    }")
        L.append("}")
        return "\n".join(L), args

    # ---------------- row mode ----------------
    # "row": a workgroup owns one row, lanes walk along it.
    # "col": rows are unit-stride neighbours in memory (a reduction down the
    #        columns of a row-major matrix): a workgroup owns 64 adjacent rows,
    #        one per lane, so every wavefront load is one contiguous run; the
    #        wavefronts of the workgroup split the reduction axis and combine in LDS.
    col_mode = spec.mode == "col"
    rng_strided = True
    L.append("    const int lane = tid & 63, wave = tid >> 6;")
    if col_mode:
        L.append("    const long row_raw = (long)blockIdx.x * 64 + lane;")
        L.append("    const bool active = row_raw < rows;")
        L.append("    const long row = active ? row_raw : rows - 1;")
        L.append("    __shared__ float red_f[THREADS];")
        L.append("    __shared__ int red_i[THREADS];")
    else:
        L.append("    const long row = blockIdx.x;")
        L.append("    if (row >= rows) return;")
        L.append("    const bool active = true;")
        L.append("    __shared__ float red_f[THREADS / 64 + 1];")
        L.append("    __shared__ int red_i[THREADS / 64 + 1];")
    L.append("    (void)lane; (void)wave; (void)red_f; (void)red_i; (void)active;")
    for t in spec.tensors:
        arg_id, code, access, take_axis, is_out = t
        if take_axis == 1:
            L.append("    p%d += (long)take%d[row] * rs%d;" % (arg_id, arg_id, arg_id))
        else:
            L.append("    p%d += row * rs%d;" % (arg_id, arg_id))
        if access == "row" and not is_out:
            L.append("    const float x%d_row = (float)p%d[0];" % (arg_id, arg_id))
    for s in range(spec.n_onehot):
        L.append("    const int oh%d_row = oh%d[row]; (void)oh%d_row;" % (s, s, s))
    for c in consts:
        em.names[("c", c)] = "c%d" % c

    loaded = set()

    def loop_open(bound):
        if col_mode:
            if ITEMS:
                return ["    _Pragma(\"unroll\") for (int it = 0; it < %d; it++) {" % ITEMS,
                        "        const int col = it * (THREADS / 64) + wave;",
                        "        if (col < %s) {" % bound]
            return ["    _Pragma(\"unroll 8\") for (int col = wave; col < %s; col += THREADS / 64) {" % bound, "        {"]
        if ITEMS:
            return ["    _Pragma(\"unroll\") for (int it = 0; it < %d; it++) {" % ITEMS,
                    "        const int col = (it * THREADS + tid) * VEC;",
                    "        if (col < %s) {" % bound]
        return ["    for (int col = tid * VEC; col < %s; col += THREADS * VEC) {" % bound, "        {"]

    def needed_tensors(node, acc):
        if node.kind == "tensor":
            acc.add(node.arg_id)
        if node.kind != "red":
            for a in node.args:
                needed_tensors(a, acc)
        return acc

    cached = bool(ITEMS)
    if cached:
        # read every streamed operand once into registers
        for t in in_ts:
            if t[2] == "row":
                continue
            L.append("    float x%d_c[%d][%d];" % (t[0], ITEMS, V))
        L += loop_open("n")
        for t in in_ts:
            if t[2] == "row":
                continue
            tmp = []
            _gen_load(spec, t, "l", "col", tmp, 12)
            L += tmp
            L.append("            _Pragma(\"unroll\") for (int v = 0; v < %d; v++) x%d_c[it][v] = x%d_l[v];" % (V, t[0], t[0]))
        L.append("        }")
        L.append("    }")

    def tensor_val(arg_id, item, v):
        t = spec._tensor_by_id[arg_id]
        if t[2] == "row":
            return "x%d_row" % arg_id
        if cached:
            return "x%d_c[it][%s]" % (arg_id, v)
        return "x%d_l[%s]" % (arg_id, v)
    spec.tensor_value = tensor_val

    def block_reduce(kind, var, ivar=None):
        o = []
        comb = {"sum": "{0} += {1};", "max": "{0} = fmaxf({0}, {1});", "min": "{0} = fminf({0}, {1});"}
        if col_mode:
            # lanes are different rows: combine the wavefronts' partials only
            if T == 64:
                return o
            if kind in comb:
                o.append("    __syncthreads(); red_f[tid] = %s; __syncthreads();" % var)
                o.append("    %s = red_f[lane];" % var)
                o.append("    _Pragma(\"unroll\") for (int w = 1; w < THREADS / 64; w++) { const float o_ = red_f[w * 64 + lane]; %s }"
                         % comb[kind].format(var, "o_"))
            else:
                better = ">" if kind == "argmax" else "<"
                merge = ("if (o_ %s %s || (o_ == %s && oi_ >= 0 && (oi_ < %s || %s < 0))) { %s = o_; %s = oi_; }"
                         % (better, var, var, ivar, ivar, var, ivar))
                o.append("    __syncthreads(); red_f[tid] = %s; red_i[tid] = %s; __syncthreads();" % (var, ivar))
                o.append("    %s = red_f[lane]; %s = red_i[lane];" % (var, ivar))
                o.append("    _Pragma(\"unroll\") for (int w = 1; w < THREADS / 64; w++) { const float o_ = red_f[w * 64 + lane]; const int oi_ = red_i[w * 64 + lane]; %s }" % merge)
            return o
        if kind in comb:
            o.append("    _Pragma(\"unroll\") for (int off = 32; off > 0; off >>= 1) { const float o_ = __shfl_xor(%s, off, 64); %s }"
                     % (var, comb[kind].format(var, "o_")))
            if T > 64:
                o.append("    __syncthreads(); if (lane == 0) red_f[wave] = %s; __syncthreads();" % var)
                o.append("    %s = red_f[0];" % var)
                o.append("    _Pragma(\"unroll\") for (int w = 1; w < THREADS / 64; w++) { const float o_ = red_f[w]; %s }"
                         % comb[kind].format(var, "o_"))
        else:
            better = ">" if kind == "argmax" else "<"
            merge = ("if (o_ %s %s || (o_ == %s && oi_ >= 0 && (oi_ < %s || %s < 0))) { %s = o_; %s = oi_; }"
                     % (better, var, var, ivar, ivar, var, ivar))
            o.append("    _Pragma(\"unroll\") for (int off = 32; off > 0; off >>= 1) { const float o_ = __shfl_xor(%s, off, 64); const int oi_ = __shfl_xor(%s, off, 64); %s }"
                     % (var, ivar, merge))
            if T > 64:
                o.append("    __syncthreads(); if (lane == 0) { red_f[wave] = %s; red_i[wave] = %s; } __syncthreads();" % (var, ivar))
                o.append("    %s = red_f[0]; %s = red_i[0];" % (var, ivar))
                o.append("    _Pragma(\"unroll\") for (int w = 1; w < THREADS / 64; w++) { const float o_ = red_f[w]; const int oi_ = red_i[w]; %s }" % merge)
        return o

    for lvl in levels:
        stage = [r for r in reds if r.level == lvl]
        pre = []
        for r in stage:
            em.prepare_scalars(r.args[0], pre, lvl - 1)
        L += pre
        for r in stage:
            var = em.fresh("red")
            r.extra = var
            if r.name == "sum":
                L.append("    float %s = 0.0f;" % var)
            elif r.name == "max":
                L.append("    float %s = -3.402823466e+38f;" % var)
            elif r.name == "min":
                L.append("    float %s = 3.402823466e+38f;" % var)
            elif r.name == "argmax":
                L.append("    float %s = -3.402823466e+38f; int %s_i = -1;" % (var, var))
            else:
                L.append("    float %s = 3.402823466e+38f; int %s_i = -1;" % (var, var))
        L += loop_open("n")
        if not cached:
            need = set()
            for r in stage:
                needed_tensors(r.args[0], need)
            for t in in_ts:
                if t[0] in need and t[2] != "row":
                    tmp = []
                    _gen_load(spec, t, "l", "col", tmp, 12)
                    L += tmp
        if need_idx:
            L.append("            const unsigned rng_idx = (unsigned)row * rng_rm + (unsigned)col * rng_cm; (void)rng_idx;")
        for v in range(V):
            # vectors are only used when they divide the row, so a vector that
            # starts inside the row lies inside it entirely
            L.append("            {")
            local, blk = {}, []
            for r in stage:
                val = em.emit_elem(r.args[0], blk, local, "it", str(v)) if not r.args[0].scalar \
                    else em.names[r.args[0].key]
                var = r.extra
                if r.name == "sum":
                    blk.append("            %s += %s;" % (var, val))
                elif r.name == "max":
                    blk.append("            %s = fmaxf(%s, %s);" % (var, var, val))
                elif r.name == "min":
                    blk.append("            %s = fminf(%s, %s);" % (var, var, val))
                elif r.name == "argmax":
                    blk.append("            if (%s > %s) { %s = %s; %s_i = col + %d; }" % (val, var, var, val, var, v))
                else:
                    blk.append("            if (%s < %s) { %s = %s; %s_i = col + %d; }" % (val, var, var, val, var, v))
            L += ["    " + b for b in blk]
            L.append("            }")
        L.append("        }")
        L.append("    }")
        for r in stage:
            var = r.extra
            if r.name in ("argmax", "argmin"):
                L += block_reduce(r.name, var, var + "_i")
                res = em.fresh("s")
                L.append("    const float %s = (float)%s_i;" % (res, var))
                em.names[r.key] = res
            else:
                L += block_reduce(r.name, var)
                em.names[r.key] = var

    # final stage
    pre = []
    em.prepare_scalars(root, pre, max(levels + [0]))
    L += pre
    if red_out:
        val = em.emit_scalar_tree(root, L)
        arg_id, code = out_t[0], out_t[1]
        L.append("    if (%s) {" % ("wave == 0 && active" if col_mode else "tid == 0"))
        L.append("        const unsigned rng_idx = (unsigned)row * rng_rm; (void)rng_idx;")
        L.append("        p%d[0] = %s;" % (arg_id, _gen_round(code, val, rounding, "rng_idx")))
        L.append("    }")
    else:
        L += loop_open("n_out")
        if not cached:
            need = needed_tensors(root, set())
            for t in in_ts:
                if t[0] in need and t[2] != "row":
                    tmp = []
                    _gen_load(spec, t, "l", "col", tmp, 12, "n_out")
                    L += tmp
        L.append("            const unsigned rng_idx = (unsigned)row * rng_rm + (unsigned)col * rng_cm; (void)rng_idx;")
        vals = []
        for v in range(V):
            local, blk = {}, []
            if root.scalar:
                vals.append(em.emit_scalar_tree(root, blk))
            else:
                vals.append(em.emit_elem(root, blk, local, "it", str(v)))
            L += blk
        L += store_code("it", "col", vals, 12)
        L.append("        }")
        L.append("    }")
    L.append("}")
    return "\n".join(L), args


# ---------------------------------------------------------------------------
# host side: marshal a postfix stack into a kernel spec + launch arguments
# ---------------------------------------------------------------------------

_kernel_cache = {}


def _get_kernel(spec):
    hit = _kernel_cache.get(spec.key)
    if hit is None:
        name = "ew_%d" % len(_kernel_cache)
        source, arg_order = generate_source(spec, name)
        module = _lib.Module(source, name)
        hit = (module.get_function(name), arg_order, source)
        _kernel_cache[spec.key] = hit
    return hit


def _pow2_at_least(x):
    p = 1
    while p < x:
        p *= 2
    return p


class _Plan(object):
    """Result of analysing one expression stack: kernel spec + argument values."""
    pass


def _is_number(arg):
    return type(arg) in (int, float) or isinstance(arg, (np.integer, np.floating))


def _stack_traits(args, tensor_type):
    """One look at a postfix stack: (axis, reduces, native_2d).

    axis       the one axis every reduction of the stack runs along (1 without reductions);
               a stack that reduces along two different axes, or along none, is refused
               (nervanagpu/float_ew.py:1090-1103)
    native_2d  the kernel has to see the operands' own rows and columns, because something in
               the stack depends on them: a reduction, a one-hot generator, an operand that
               broadcasts (fewer than two dimensions or a unit extent), a transposed view, a
               fancy-index view or a view with gaps.  Otherwise every operand is just `size`
               consecutive values (nervanagpu/float_ew.py:1104-1137)."""
    ops = [a for a in args if type(a) is dict]
    axes = set(a.get("axis", None) for a in ops if a["op"] in _reduction_ops)
    if axes - set((0, 1)):
        raise ValueError("Only reduction along an axis currently supported")
    if len(axes) > 1:
        raise ValueError("Reduction only allowed along one axis per kernel.")
    reduces = bool(axes)
    axis = axes.pop() if reduces else 1

    def own_geometry(t):
        thin = len(t.shape) < 2 or (len(t.shape) == 2 and 1 in t.shape)
        return thin or t.is_trans or bool(t.take_array) or not t.is_contiguous

    native_2d = (reduces or any(a["op"] == "onehot" for a in ops) or
                 any(own_geometry(a) for a in args if isinstance(a, tensor_type)))
    return axis, reduces, native_2d


class _Extents(object):
    """The (rows, columns) extents of the partial results while a postfix stack is walked:
    operands push theirs, an operator replaces those of its inputs by their broadcast."""

    def __init__(self):
        self.pending = []
        self.widest = [1, 1]       # broadcast of the last operator's inputs

    def push(self, extent):
        self.pending.append(tuple(extent))

    def join(self, count):
        joined = [1, 1]
        for _ in range(count):
            extent = self.pending.pop()
            for d in (0, 1):
                if extent[d] == joined[d] or extent[d] == 1:
                    continue
                if joined[d] != 1:
                    raise TypeError("Input shape:%s not compatible" % (extent,))
                joined[d] = extent[d]
        self.widest = joined
        return tuple(joined)

    def collapse(self, axis):
        """a reduction along `axis`: returns the reduced depth"""
        extent = list(self.pending.pop())
        depth = extent[axis]
        extent[axis] = 1
        self.pending.append(tuple(extent))
        return depth


def _kept_mantissa_bits(out):
    """stochastic-rounding width of a store into `out` (0: nearest): True means the full
    fp16 mantissa; clamped to [1, 10] for fp16 and [1, 15] for fp32
    (nervanagpu/float_ew.py:1225-1237); integer outputs always round to nearest"""
    bits = out.rounding
    if not bits or out.dtype.kind != "f":
        return 0
    if bits is True:
        bits = 10
    cap = {np.float32: 15, np.float16: 10}.get(out.dtype.type)
    if cap is not None:
        bits = min(bits, cap)
    return max(int(bits), 1)


def analyse(args):
    """Shape / stride / broadcast analysis of a postfix stack: what
    call_compound_kernel works out before it asks for a kernel
    (nervanagpu/float_ew.py:1058-1286).  Pure host logic: needs no GPU, tensors
    only need .shape/.strides/.dtype/.size/.is_trans/.take_array/
    .is_contiguous/.gpudata/.rounding.

    Kernel arguments are numbered in order of first appearance.  The first tensor
    of the stack is the output and always takes argument 0; if the same tensor
    occurs again it is an input and gets an argument of its own (an in-place
    expression reads through a const pointer, nervanagpu/float_ew.py:1145-1154).
    Every other tensor, and every distinct constant, is passed once."""
    from .nervanagpu import GPUTensor

    axis, reduction, complex_op = _stack_traits(args, GPUTensor)

    plan = _Plan()
    type_args = []
    values = {}                    # kernel argument number -> what is passed there
    slot_of_tensor, slot_of_const = {}, {}
    out = None
    extents = _Extents()
    onehots, onehot_pos = [], []
    flat_size = None
    red_depth = 0
    n_ops = 0

    def geometry(t):
        """(extent, [row stride, column stride]) as the kernel sees operand t; with
        reductions down the columns (axis 0) rows and columns swap roles in the
        strides, so that the kernel always walks along its second stride"""
        if not complex_op:
            return (1, t.size), [0, 1]
        if len(t.shape) == 2:
            extent = tuple(t.shape)
            strides = [t.strides[0], t.strides[1]]
        elif len(t.shape) < 2:
            # 0-d / 1-d operands broadcast as a row vector
            extent = (1, t.size)
            strides = [0, t.strides[0] if t.strides else 0]
        else:
            raise ValueError("Operations that are not simple elementwise are only currently supported in 2 dimensions.")
        if axis == 0:
            strides.reverse()
        # a unit extent broadcasts: never step along it
        if extent[0] == 1:
            strides[1 - axis] = 0
        if extent[1] == 1:
            strides[axis] = 0
        return extent, strides

    for pos, arg in enumerate(args):
        if isinstance(arg, GPUTensor):
            extent, strides = geometry(arg)
            if not complex_op:
                if flat_size is None:
                    flat_size = arg.size
                elif flat_size != arg.size:
                    raise TypeError("Input shape:%s not compatible" % (arg.shape,))
            is_out = out is None
            if is_out:
                out = arg
                slot = len(values)
            else:
                slot = slot_of_tensor.get(id(arg))
                if slot is None:
                    slot = slot_of_tensor[id(arg)] = len(values)
            if slot not in values:
                take_axis, take_ptr = 0, None
                if arg.take_array:
                    take_axis = (2 - arg.take_array[1]) if axis != 1 else (arg.take_array[1] + 1)
                    take_ptr = arg.take_array[0].gpudata
                values[slot] = dict(ptr=int(arg.gpudata) if arg.gpudata is not None else 0,
                                    rs=int(strides[0]), cs=int(strides[1]), take=take_ptr,
                                    dtype=arg.dtype.str[1:], take_axis=take_axis, is_out=is_out,
                                    itemsize=arg.dtype.itemsize, pos=pos)
            type_args.append(("tensor", slot))
            extents.push(extent)

        elif _is_number(arg):
            val = float(arg)
            slot = slot_of_const.get(val)
            if slot is None:
                slot = slot_of_const[val] = len(values)
                values[slot] = dict(const=val, pos=pos)
            type_args.append(("const", slot))
            extents.push((1, 1))

        elif type(arg) is dict:
            op_name = arg["op"]
            if op_name in _float_ops:
                had_inputs = bool(extents.pending)
                joined = extents.join(_float_ops[op_name][0])
                if op_name == "assign":
                    plan.rounding = _kept_mantissa_bits(out)
                    type_args.append(("assign", n_ops, plan.rounding > 0))
                elif op_name == "onehot":
                    hot_axis = arg["axis"] if axis else 1 - arg["axis"]
                    type_args.append(("onehot", n_ops, hot_axis, len(onehots)))
                    onehots.append(arg["idx"].gpudata)
                    onehot_pos.append(pos)
                    extents.push(joined if had_inputs else (1, 1))
                else:
                    type_args.append((op_name, n_ops))
                    extents.push(joined)
            elif op_name in _reduction_ops:
                type_args.append((op_name, n_ops))
                red_depth = max(red_depth, extents.collapse(axis))
            else:
                raise TypeError("%s is not a valid operation" % op_name)
            n_ops += 1
        else:
            raise TypeError("args must be instance of GPUTensor, int, float, or dict (for operators)")

    max_shape = extents.widest

    if out is None:
        raise TypeError("expression has no output tensor")

    plan.out = out
    plan.axis = axis
    plan.values = values
    plan.onehots = onehots
    plan.onehot_pos = onehot_pos
    plan.type_args = type_args

    if not complex_op:
        size = out.size
        plan.mode = "flat"
        # output shape is the broadcast target: assigning a constant is allowed
        ptr_or = 0
        for v in values.values():
            if "ptr" in v:
                ptr_or |= v["ptr"]
        vec = 1
        for cand in (8, 4, 2):
            ok = size % cand == 0
            for v in values.values():
                if "ptr" in v and (v["ptr"] % min(cand * v["itemsize"], 16)) != 0:
                    ok = False
            if ok:
                vec = cand
                break
        plan.vec = vec
        plan.n = plan.n_out = size
        plan.rows = size // vec
        plan.threads = 256
        plan.items = 0
        per_block = 256 * FLAT_UNROLL
        plan.grid = max(1, min((plan.rows + per_block - 1) // per_block, 16384))
        plan.rng_rm, plan.rng_cm = 0, 1
        tensors = [(i, v["dtype"], "vec", 0, v["is_out"]) for i, v in sorted(values.items()) if "ptr" in v]
    else:
        # the output may be a broadcast target of the expression, never smaller
        out_shape = tuple(out.shape) if len(out.shape) == 2 else (1, out.size)
        for i in range(2):
            if max_shape[i] not in (1, out_shape[i]) and out_shape[i] != 1:
                raise TypeError("Input shape:%s not compatible" % (tuple(max_shape),))
        full = [max(max_shape[i], out_shape[i]) for i in range(2)]
        n_out = full[axis]
        n = red_depth if reduction else n_out
        rows = full[1 - axis]
        plan.mode = "row"
        plan.n, plan.n_out, plan.rows = n, n_out, rows
        # logical flat index of (row, col) in the output tensor for the random stream
        ncols_out = out_shape[1]
        if axis == 1:
            plan.rng_rm, plan.rng_cm = ncols_out, 1
        else:
            plan.rng_rm, plan.rng_cm = 1, ncols_out
        vec = 1
        for cand in (8, 4, 2):
            ok = n % cand == 0 and (n_out % cand == 0 or n_out == 1)
            for v in values.values():
                if "ptr" not in v:
                    continue
                if v["take_axis"]:
                    continue
                if v["cs"] == 1:
                    width = min(cand * v["itemsize"], 16)
                    if v["ptr"] % width or (v["rs"] * v["itemsize"]) % width:
                        ok = False
            if ok:
                vec = cand
                break
        if not any(("ptr" in v and v["cs"] == 1 and not v["take_axis"]) for v in values.values()):
            vec = 1
        plan.vec = vec
        nvec = (max(n, n_out) + vec - 1) // vec
        streamed = [v for v in values.values() if "ptr" in v and (v["cs"] != 0 or v["is_out"])]
        col_mode = (vec == 1 and rows >= 32 and not any(v["take_axis"] for v in values.values() if "ptr" in v)
                    and all(v["rs"] in (0, 1) for v in values.values() if "ptr" in v)
                    and any(v["rs"] == 1 for v in streamed))
        if col_mode:
            # neighbouring rows are adjacent in memory: one row per lane, the
            # wavefronts of a workgroup share the walk along the row
            plan.mode = "col"
            groups = min(16, max(1, _pow2_at_least((nvec + 7) // 8)))
            threads = 64 * groups
            items = (nvec + groups - 1) // groups
            plan.grid = (rows + 63) // 64
        else:
            threads = min(MAX_THREADS, max(64, _pow2_at_least((nvec + 3) // 4)))
            if not reduction:
                threads = min(threads, 256)
            items = (nvec + threads - 1) // threads
            plan.grid = rows
        # keep the row in registers only when every loop walks the same extent
        if items * vec > MAX_CACHED_PER_LANE or not reduction or n_out not in (1, n):
            items = 0
        plan.threads, plan.items = threads, items
        tensors = []
        for i, v in sorted(values.items()):
            if "ptr" not in v:
                continue
            if v["take_axis"]:
                access = "strided"
            elif v["cs"] == 0 and not v["is_out"]:
                access = "row"
            elif v["cs"] == 1 and vec > 1:
                access = "vec"
            else:
                access = "strided"
            tensors.append((i, v["dtype"], access, v["take_axis"], v["is_out"]))

    rng_pair = plan.vec > 1 and plan.rng_cm == 1 and plan.rng_rm % 2 == 0
    plan.spec = KernelSpec(type_args, tensors, plan.mode, plan.vec, plan.threads, plan.items, len(onehots), rng_pair)
    return plan


_GPUTensor = None


def _signature(args):
    """Everything about a postfix stack that the analysis depends on, leaving out
    what is merely passed through to the kernel (addresses, constant values)."""
    global _GPUTensor
    if _GPUTensor is None:
        from .nervanagpu import GPUTensor as _T
        _GPUTensor = _T
    GPUTensor = _GPUTensor
    sig = []
    tensors, consts = {}, {}
    for arg in args:
        if type(arg) is dict:
            sig.append((arg["op"], arg.get("axis", None)))
        elif isinstance(arg, GPUTensor):
            key = id(arg)
            slot = tensors.get(key)
            if slot is None:
                slot = tensors[key] = len(tensors)
                take = arg.take_array
                base = arg.gpudata
                sig.append((slot, arg.shape, arg.strides, arg.dtype.char, arg.is_trans,
                            arg.rounding if slot == 0 else 0,
                            take[1] if take else None,
                            (int(base) & 15) if base is not None else 0))
            else:
                sig.append(slot)
        elif type(arg) in (int, float) or isinstance(arg, (np.integer, np.floating)):
            val = float(arg)
            slot = consts.get(val)
            if slot is None:
                slot = consts[val] = len(consts)
            sig.append(("c", slot))
        else:
            raise TypeError("args must be instance of GPUTensor, int, float, or dict (for operators)")
    return tuple(sig)


class _BoundLaunch(object):
    """A compiled kernel with a persistent argument block.  Structurally identical
    expressions reuse it; a call only patches the values that may differ between
    them: addresses, constants and the random stream."""

    _PTR, _TAKE, _CONST, _ONEHOT = range(4)

    def __init__(self, plan, func, arg_order):
        self.func = func
        self.grid = (c_uint * 3)(plan.grid, 1, 1)
        self.block = (c_uint * 3)(plan.threads, 1, 1)
        self.empty = plan.rows == 0 or plan.n == 0
        self.uses_rng = bool(plan.rounding) or any(a[0] == "rand" for a in plan.type_args)
        self.shape = (plan.rows, plan.n, plan.grid, plan.threads)
        self.patches = []
        self.c_seed = c_uint(0)
        self.c_stream = c_uint(0)
        cargs = []
        for a in arg_order:
            kind = a[0]
            if kind == "ptr":
                c = c_void_p(plan.values[a[1]]["ptr"])
                self.patches.append((c, self._PTR, plan.values[a[1]]["pos"]))
            elif kind == "rs":
                c = c_int(plan.values[a[1]]["rs"])
            elif kind == "cs":
                c = c_int(plan.values[a[1]]["cs"])
            elif kind == "take":
                c = c_void_p(int(plan.values[a[1]]["take"]))
                self.patches.append((c, self._TAKE, plan.values[a[1]]["pos"]))
            elif kind == "const":
                c = c_float(plan.values[a[1]]["const"])
                self.patches.append((c, self._CONST, plan.values[a[1]]["pos"]))
            elif kind == "onehot":
                c = c_void_p(int(plan.onehots[a[1]]))
                self.patches.append((c, self._ONEHOT, plan.onehot_pos[a[1]]))
            elif kind == "n":
                c = c_int(plan.n)
            elif kind == "n_out":
                c = c_int(plan.n_out)
            elif kind == "rows":
                c = ctypes.c_long(plan.rows)
            elif kind == "sr_bits":
                c = c_uint(plan.rounding)
            elif kind == "rng_seed":
                c = self.c_seed
            elif kind == "rng_stream":
                c = self.c_stream
            elif kind == "rng_rm":
                c = c_uint(plan.rng_rm)
            elif kind == "rng_cm":
                c = c_uint(plan.rng_cm)
            else:
                raise AssertionError(kind)
            cargs.append(c)
        self.cargs = cargs          # keeps the storage the pointer block refers to alive
        self.ptrs = (c_void_p * len(cargs))(*[ctypes.addressof(c) for c in cargs])
        self.entry = _lib.load().ng_launch

    def __call__(self, backend, args):
        if self.empty:
            return
        for c, kind, pos in self.patches:
            a = args[pos]
            if kind == 0:
                base = a.gpudata
                c.value = int(base) if base is not None else 0
            elif kind == 2:
                c.value = float(a)
            elif kind == 1:
                c.value = int(a.take_array[0].gpudata)
            else:
                c.value = int(a["idx"].gpudata)
        if self.uses_rng:
            self.c_seed.value, self.c_stream.value = backend._next_rng_stream()
        repeat = backend.bench if isinstance(backend.bench, int) and backend.bench > 1 else 1
        if repeat > 1:
            start, end = backend._get_events()
            start.record(backend.stream)
        for _ in range(repeat):
            _lib.check(self.entry(self.func.handle, self.grid, self.block, 0, backend.stream, self.ptrs))
        if repeat > 1:
            end.record(backend.stream)
            end.synchronize()
            msecs = end.time_since(start) / repeat
            backend.last_bench_msecs = msecs
            print("%7.3f msecs shape(%d,%d) blk,thd(%d,%d) %s" % ((msecs,) + self.shape + (self.func.name,)))


_bound_cache = {}


def call_compound_kernel(backend, *args):
    """Execute a postfix expression stack ending in {"op": "assign"}:
        C += 2.5 * A * B + 1  ==  (C, 2.5, A, mul, B, mul, 1, add, C, add, assign)
    `backend` supplies the stream and the random stream (seed, launch counter).
    Returns the output tensor (nervanagpu/float_ew.py:1058-1322)."""
    sig = _signature(args)
    bound = _bound_cache.get(sig)
    if bound is None:
        plan = analyse(args)
        if plan.rows == 0 or plan.n == 0:
            return plan.out
        func, arg_order, _ = _get_kernel(plan.spec)
        bound = _bound_cache[sig] = _BoundLaunch(plan, func, arg_order)
    bound(backend, args)
    return args[0]


# ---------------------------------------------------------------------------
# Kahan-compensated accumulate: one kernel, three reads and two writes
# ---------------------------------------------------------------------------

_compensated_sum_cache = {}


def compensated_sum_source(code, stochastic, name="compensated_sum"):
    """HIP source of  y = add*add_scale - cmp*cmp_scale;  t = round(sum + y);
    cmp = round_nearest((t - sum) - y);  sum = t   on 2-D strided tensors
    (the arithmetic of nervanagpu/float_ew.py:1453-1475: every step in fp32, the
    running sum rounded like its tensor, the error term always to nearest).
    Contiguous tensors run as one row of 8-element vectors; element e = row *
    cols + col draws word e of the random stream."""
    ct = _ctype(code)
    idx = "(unsigned)(i + v)"
    src = [_lib.common_header_text(), ""]
    src.append('extern "C" __global__ __launch_bounds__(256)')
    src.append("void %s(%s* __restrict__ sum, %s* __restrict__ cmp, const %s* __restrict__ add," % (name, ct, ct, ct))
    src.append("        float cmp_scale, float add_scale, long n, int cols, int vec,")
    src.append("        long rs_sum, long cs_sum, long rs_cmp, long cs_cmp, long rs_add, long cs_add,")
    src.append("        unsigned sr_bits, unsigned rng_seed, unsigned rng_stream)")
    src.append("{")
    src.append("    const long stride = (long)gridDim.x * 256 * 8;")
    src.append("    for (long i = ((long)blockIdx.x * 256 + threadIdx.x) * 8; i < n; i += stride) {")
    src.append("        %s s[8], c[8], a[8];" % ct)
    src.append("        long os[8], oc[8];")
    src.append("        if (vec) {")
    src.append("            typedef %s vt_ __attribute__((ext_vector_type(8)));" % ct)
    src.append("            *reinterpret_cast<vt_*>(s) = *reinterpret_cast<const vt_*>(sum + i);")
    src.append("            *reinterpret_cast<vt_*>(c) = *reinterpret_cast<const vt_*>(cmp + i);")
    src.append("            *reinterpret_cast<vt_*>(a) = *reinterpret_cast<const vt_*>(add + i);")
    src.append("        } else {")
    src.append('            _Pragma("unroll") for (int v = 0; v < 8; v++) {')
    src.append("                const long e = (i + v < n) ? i + v : n - 1;")
    src.append("                const long r = e / cols, q = e - r * cols;")
    src.append("                os[v] = r * rs_sum + q * cs_sum; oc[v] = r * rs_cmp + q * cs_cmp;")
    src.append("                s[v] = sum[os[v]]; c[v] = cmp[oc[v]]; a[v] = add[r * rs_add + q * cs_add];")
    src.append("            }")
    src.append("        }")
    src.append('        _Pragma("unroll") for (int v = 0; v < 8; v++) {')
    src.append("            const float s32 = (float)s[v];")
    src.append("            const float y32 = (float)a[v] * add_scale - (float)c[v] * cmp_scale;")
    src.append("            const %s t = %s;" % (ct, _gen_round(code, "(s32 + y32)", stochastic, idx)))
    src.append("            c[v] = %s;" % _gen_round(code, "(((float)t - s32) - y32)", 0, idx))
    src.append("            s[v] = t;")
    src.append("        }")
    src.append("        if (vec) {")
    src.append("            typedef %s vt_ __attribute__((ext_vector_type(8)));" % ct)
    src.append("            *reinterpret_cast<vt_*>(sum + i) = *reinterpret_cast<const vt_*>(s);")
    src.append("            *reinterpret_cast<vt_*>(cmp + i) = *reinterpret_cast<const vt_*>(c);")
    src.append("        } else {")
    src.append('            _Pragma("unroll") for (int v = 0; v < 8; v++)')
    src.append("                if (i + v < n) { sum[os[v]] = s[v]; cmp[oc[v]] = c[v]; }")
    src.append("        }")
    src.append("    }")
    src.append("}")
    return "\n".join(src)


def call_compensated_sum(backend, sum_tensor, cmp_tensor, add_tensor, cmp_scale, add_scale):
    """launch the fused accumulate on three tensors of one shape and dtype
    (at most two dimensions unless all are contiguous)"""
    code = sum_tensor.dtype.str[1:]
    assert code in ("f2", "f4"), "compensated_sum works on fp16 or fp32 tensors"
    assert sum_tensor.shape == cmp_tensor.shape == add_tensor.shape
    tensors = (sum_tensor, cmp_tensor, add_tensor)
    assert not any(t.take_array for t in tensors)
    rounding = int(sum_tensor.rounding or 0)
    sr_bits = max(1, min(rounding, 10 if code == "f2" else 15)) if rounding else 0
    key = (code, bool(rounding))
    fn = _compensated_sum_cache.get(key)
    if fn is None:
        name = "compensated_sum_%s_%s" % (code, "sr" if rounding else "rn")
        fn = _lib.Module(compensated_sum_source(code, bool(rounding), name), name).get_function(name)
        _compensated_sum_cache[key] = fn
    n = sum_tensor.size
    if n == 0:
        return sum_tensor
    es = sum_tensor.dtype.itemsize
    flat = all(t.is_contiguous for t in tensors)
    vec = int(flat and n % 8 == 0 and all(int(t.gpudata) % (8 * es) == 0 for t in tensors))
    if flat:
        cols, strides = n, [(0, 1)] * 3
    else:
        assert len(sum_tensor.shape) == 2, "strided operands of compensated_sum must be two-dimensional"
        cols, strides = sum_tensor.shape[1], [tuple(t.strides) for t in tensors]
    seed, stream_id = backend._next_rng_stream() if rounding else (0, 0)
    cus = _lib.device_attr(0)
    blocks = max(1, min((n + 2047) // 2048, cus * 8))
    args = [c_void_p(int(sum_tensor.gpudata)), c_void_p(int(cmp_tensor.gpudata)), c_void_p(int(add_tensor.gpudata)),
            c_float(cmp_scale), c_float(add_scale), c_long(n), c_int(cols), c_int(vec)]
    for rs, cs in strides:
        args += [c_long(rs), c_long(cs)]
    args += [c_uint(sr_bits), c_uint(seed), c_uint(stream_id)]
    fn.launch((blocks, 1, 1), (256, 1, 1), backend.stream, args)
    return sum_tensor
