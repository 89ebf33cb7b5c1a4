"""HIP kernel source generators for gfx950 (MI355X, CDNA4, wave64).

Counterpart of dlgrad/codegen/cpu_kernel.py: every function returns
`(source, kernel_name, argfmt)` where `argfmt` is the `struct` format of the
kernel's argument block.  The sources are compiled by hiprtc at first use (or
ahead of time by the build step) and cached as code objects.

Specialisation is by *layout class*, not by exact shape: the element-wise
generator, for example, is instantiated per (expression, operand modes, vector
width), and sizes are runtime arguments.  That keeps the set of code objects
finite so all of them can be built ahead of time, while the launch code still
picks the variant that matches the shape at hand (vector width by divisibility
and alignment, tile shape by problem size).

Kernel families
  map_kernel            element-wise n-ary op over a contiguous output; operands are
                        same-shape, scalar (by value or from memory), row-broadcast
                        (one value per row) or column-broadcast (one row repeated)
  strided_map_kernel    the same for arbitrary <=4-D broadcast strides
  reduce_full/rows/cols sum, max, mean and arg-max reductions
  permute_rows/tiled    materialised permutations
  matmul_kernel         LDS-tiled fp32 MFMA GEMM, batched and broadcast by stride
  embedding_*           gather and atomic scatter-add
  ce_*, softmax_rows    cross-entropy helpers and fused row softmax
"""
from __future__ import annotations

from functools import cache

ARCH = "gfx950"
# -packed-fp32-ops is switched off on purpose: hipcc -O3 otherwise forms
# v_pk_{add,mul,fma}_f32 from plain float code.
COMPILE_OPTIONS = (
    f"--offload-arch={ARCH}", "-O3", "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
)

WAVE = 64

PRELUDE = r"""
typedef unsigned int u32;
typedef unsigned long long u64;
typedef float v4f __attribute__((ext_vector_type(4)));
#define WAVE 64
#define NEG_FLT_MAX (-3.402823466e+38f)
// 16-byte load that does not displace cached data (inputs streamed once)
static __device__ __forceinline__ float4 ld4_stream(const float4* p) {
    const v4f t = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(p));
    return make_float4(t.x, t.y, t.z, t.w);
}

// ---- wavefront-64 reductions: DPP inside each row of 16 lanes, then two
// cross-row exchanges.  After the call every lane holds the result.
#define DPP_XOR1        0xB1   /* quad_perm:[1,0,3,2] */
#define DPP_XOR2        0x4E   /* quad_perm:[2,3,0,1] */
#define DPP_HALF_MIRROR 0x141  /* row_half_mirror     */
#define DPP_MIRROR      0x140  /* row_mirror          */
template <int CTRL> static __device__ __forceinline__ float dpp_f(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, false));
}
static __device__ __forceinline__ float wave_sum(float v) {
    v += dpp_f<DPP_XOR1>(v);
    v += dpp_f<DPP_XOR2>(v);
    v += dpp_f<DPP_HALF_MIRROR>(v);
    v += dpp_f<DPP_MIRROR>(v);
    v += __shfl_xor(v, 16, WAVE);
    v += __shfl_xor(v, 32, WAVE);
    return v;
}
static __device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_f<DPP_XOR1>(v));
    v = fmaxf(v, dpp_f<DPP_XOR2>(v));
    v = fmaxf(v, dpp_f<DPP_HALF_MIRROR>(v));
    v = fmaxf(v, dpp_f<DPP_MIRROR>(v));
    v = fmaxf(v, __shfl_xor(v, 16, WAVE));
    v = fmaxf(v, __shfl_xor(v, 32, WAVE));
    return v;
}
"""


def _fmt(*parts: str) -> str:
    return "@" + "".join(parts)


# =====================================================================================
# element-wise
# =====================================================================================

# Expressions are written over x0, x1, x2 (operand values), s0.. (by-value scalars)
# and i (the flat output index).  Comparisons yield 0.0f / 1.0f as the reference's C
# does (cpu_kernel.py:21-24, :663).
BINARY_EXPR = {
    "add": "x0 + x1", "sub": "x0 - x1", "mul": "x0 * x1", "div": "x0 / x1",
    "eq": "(x0 == x1) ? 1.0f : 0.0f", "gt": "(x0 > x1) ? 1.0f : 0.0f",
    "gte": "(x0 >= x1) ? 1.0f : 0.0f", "lt": "(x0 < x1) ? 1.0f : 0.0f",
    "le": "(x0 <= x1) ? 1.0f : 0.0f",
}
UNARY_EXPR = {
    "neg": "-x0",                       # c_neg: -1 * x           cpu_kernel.py:252-257
    "exp": "expf(x0)",                  # c_exp: exp() in double  cpu_kernel.py:264-269
    "log": "logf(x0)",                  # c_log: log() in double  cpu_kernel.py:276-281
    "sqrt": "sqrtf(x0)",                # c_sqrt                  cpu_kernel.py:300-305
    "rsqrt": "1.0f / sqrtf(x0)",        # c_rsqrt: 1.0/sqrtf      cpu_kernel.py:312-317
    "relu": "(x0 <= 0.0f) ? 0.0f : x0", # relu                    cpu_kernel.py:522-530
    "copy": "x0",
}


def pow_expr(n: int) -> str:
    """x0**n for an integer n by repeated squaring (c_pow receives an int exponent,
    cpu_kernel.py:288-292).  Large |n| goes through powf."""
    if n == 0:
        return "1.0f"
    if abs(n) > 64:
        return f"powf(x0, {float(n)}f)"
    # build the product from the binary digits of |n|, low bit first
    m, parts, cur = abs(n), [], "x0"
    while m:
        if m & 1:
            parts.append(cur)
        m >>= 1
        if m:
            cur = f"({cur} * {cur})"
    body = " * ".join(parts)
    return body if n > 0 else f"1.0f / ({body})"


MODES = ("vec", "sval", "sptr", "row", "col")


@cache
def map_kernel(tag: str, expr: str, modes: tuple[str, ...], vec: int, n_sval_extra: int = 0,
               unroll: int = 4, nt_store: bool = False) -> tuple[str, str, str]:
    """out[i] = expr(operands at i) over a contiguous output of n elements.

    modes[k] for operand k:
      vec   same shape as out, contiguous                     (pointer)
      sval  one value passed by value                          (float)
      sptr  one value read from memory                         (pointer)
      row   one value per row:   operand[i / C]                (pointer)
      col   one row repeated:    operand[i % C]                (pointer)
    `n_sval_extra` extra by-value floats are visible to the expression as s0, s1...
    vec=4 uses 16-byte accesses (dwordx4): the launcher guarantees 16-byte aligned
    pointers and, for row/col operands, C % 4 == 0.  The n % 4 tail is done by the
    first threads of block 0 with scalar accesses.
    nt_store: the streaming form for tensors far larger than the caches -- same-shape operands
    are read with nontemporal loads and the output is written with nontemporal stores, so
    neither evicts what the next kernel is about to read (broadcast operands, which are
    reused, keep ordinary loads).
    """
    assert vec in (1, 4) and all(m in MODES for m in modes)
    name = f"map_{tag}_{'_'.join(modes) if modes else 'gen'}_v{vec}u{unroll}{'nt' if nt_store else ''}"
    params, fmt = [], []
    for k, m in enumerate(modes):
        if m == "sval":
            params.append(f"float a{k}")
            fmt.append("f")
        else:
            params.append(f"const float* __restrict__ a{k}")
            fmt.append("P")
    # by-value scalars are packed after pointers in declaration order: keep order as declared
    for k in range(n_sval_extra):
        params.append(f"float s{k}")
        fmt.append("f")
    params += ["float* __restrict__ out", "u32 n", "u32 C"]
    fmt += ["P", "I", "I"]
    nx = len(modes)
    fargs = ", ".join([f"float x{k}" for k in range(nx)] + [f"float s{k}" for k in range(n_sval_extra)] + ["u32 i", "u32 C"])
    extra = "".join(f"s{k}, " for k in range(n_sval_extra))

    def scalar_load(k: int, idx: str) -> str:
        m = modes[k]
        return {"vec": f"a{k}[{idx}]", "sval": f"a{k}", "sptr": f"a{k}[0]",
                "row": f"a{k}[({idx}) / C]", "col": f"a{k}[({idx}) % C]"}[m]

    T = 256
    if vec == 4:
        decl = "".join(f"    float4 r{k}[{unroll}];\n" for k in range(nx) if modes[k] in ("vec", "col"))
        decl += "".join(f"    float q{k}[{unroll}];\n" for k in range(nx) if modes[k] == "row")
        pre = "".join(f"    const float c{k} = a{k}[0];\n" for k in range(nx) if modes[k] == "sptr")
        loads = ""
        for k in range(nx):
            if modes[k] == "vec":
                loads += (f"            {{ const v4f t = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(a{k}) + v); "
                          f"r{k}[u] = make_float4(t.x, t.y, t.z, t.w); }}\n" if nt_store else
                          f"            r{k}[u] = reinterpret_cast<const float4*>(a{k})[v];\n")
            elif modes[k] == "col":
                loads += f"            r{k}[u] = reinterpret_cast<const float4*>(a{k})[((v << 2) % C) >> 2];\n"
            elif modes[k] == "row":
                loads += f"            q{k}[u] = a{k}[(v << 2) / C];\n"

        def comp(k: int, c: str) -> str:
            m = modes[k]
            return {"vec": f"r{k}[u].{c}", "col": f"r{k}[u].{c}", "row": f"q{k}[u]",
                    "sval": f"a{k}", "sptr": f"c{k}"}[m]
        calc = ""
        for j, c in enumerate("xyzw"):
            xs = ", ".join([comp(k, c) for k in range(nx)])
            xs = (xs + ", ") if xs else ""
            calc += f"            o.{c} = f({xs}{extra}(v << 2) + {j}, C);\n"
        store = ("{ v4f ov = {o.x, o.y, o.z, o.w}; __builtin_nontemporal_store(ov, reinterpret_cast<v4f*>(out) + v); }" if nt_store
                 else "reinterpret_cast<float4*>(out)[v] = o;")
        tail_x = ", ".join(scalar_load(k, "i") for k in range(nx))
        tail_x = (tail_x + ", ") if tail_x else ""
        body = f"""
    const u32 nv = n >> 2;
    const u32 v0 = blockIdx.x * {T * unroll}u + threadIdx.x;
{pre}{decl}
    #pragma unroll
    for (int u = 0; u < {unroll}; ++u) {{
        const u32 v = v0 + u * {T}u;
        if (v < nv) {{
{loads}        }}
    }}
    #pragma unroll
    for (int u = 0; u < {unroll}; ++u) {{
        const u32 v = v0 + u * {T}u;
        if (v < nv) {{
            float4 o;
{calc}            {store}
        }}
    }}
    if (blockIdx.x == 0 && threadIdx.x < (n & 3u)) {{
        const u32 i = (nv << 2) + threadIdx.x;
        out[i] = f({tail_x}{extra}i, C);
    }}
"""
    else:
        xs = ", ".join(scalar_load(k, "i") for k in range(nx))
        xs = (xs + ", ") if xs else ""
        body = f"""
    const u32 i0 = blockIdx.x * {T * unroll}u + threadIdx.x;
    #pragma unroll
    for (int u = 0; u < {unroll}; ++u) {{
        const u32 i = i0 + u * {T}u;
        if (i < n) out[i] = f({xs}{extra}i, C);
    }}
"""
    src = f"""{PRELUDE}
static __device__ __forceinline__ float f({fargs}) {{ return {expr}; }}
extern "C" __global__ __launch_bounds__({T}) void {name}({', '.join(params)}) {{
{body}}}
"""
    return src, name, _fmt(*fmt)


def map_grid(n: int, vec: int, unroll: int = 4) -> int:
    per_block = 256 * unroll * vec
    return max(1, (n + per_block - 1) // per_block)


@cache
def strided_map_kernel(tag: str, expr: str, n_ops: int, sval: tuple[bool, ...],
                       n_sval_extra: int = 0) -> tuple[str, str, str]:
    """Same contract as map_kernel for operands with arbitrary broadcast strides over
    a <=4-D output (the rank-generic nested loops of cpu_kernel.py:12-66, :536-650):
    the flat output index is split into four coordinates, each operand is read at
    sum(coord*stride).  Shapes and strides are padded to 4 dims on the left."""
    name = f"smap_{tag}_{''.join('s' if s else 'p' for s in sval)}"
    params, fmt = [], []
    for k in range(n_ops):
        if sval[k]:
            params.append(f"float a{k}")
            fmt.append("f")
        else:
            params.append(f"const float* __restrict__ a{k}")
            fmt.append("P")
    for k in range(n_sval_extra):
        params.append(f"float s{k}")
        fmt.append("f")
    params += ["float* __restrict__ out", "u32 n", "Dims4 shape"]
    fmt += ["P", "I", "4I"]
    for k in range(n_ops):
        if not sval[k]:
            params.append(f"Dims4 st{k}")
            fmt.append("4I")
    fargs = ", ".join([f"float x{k}" for k in range(n_ops)] + [f"float s{k}" for k in range(n_sval_extra)] + ["u32 i"])
    loads = ", ".join(
        (f"a{k}" if sval[k] else
         f"a{k}[(u64)c0 * st{k}.d[0] + (u64)c1 * st{k}.d[1] + (u64)c2 * st{k}.d[2] + (u64)c3 * st{k}.d[3]]")
        for k in range(n_ops))
    loads = (loads + ", ") if loads else ""
    extra = "".join(f"s{k}, " for k in range(n_sval_extra))
    src = f"""{PRELUDE}
struct Dims4 {{ u32 d[4]; }};
static __device__ __forceinline__ float f({fargs}) {{ return {expr}; }}
extern "C" __global__ __launch_bounds__(256) void {name}({', '.join(params)}) {{
    const u32 i0 = blockIdx.x * 1024u + threadIdx.x;
    #pragma unroll
    for (int u = 0; u < 4; ++u) {{
        const u32 i = i0 + u * 256u;
        if (i < n) {{
            u32 r = i;
            const u32 c3 = r % shape.d[3]; r /= shape.d[3];
            const u32 c2 = r % shape.d[2]; r /= shape.d[2];
            const u32 c1 = r % shape.d[1];
            const u32 c0 = r / shape.d[1];
            out[i] = f({loads}{extra}i);
        }}
    }}
}}
"""
    return src, name, _fmt(*fmt)


# =====================================================================================
# reductions
# =====================================================================================
# (identity, combine(a, b), wave-level reduce) per op.  max starts from -FLT_MAX and
# ignores NaN, as `if (v > val) val = v` does (cpu_kernel.py:78-81, :160-163).
_RED = {
    "sum": ("0.0f", "({a} + {b})", "wave_sum"),
    "max": ("NEG_FLT_MAX", "fmaxf({a}, {b})", "wave_max"),
}

_BLOCK_REDUCE = r"""
// 256 threads = 4 waves: per-wave DPP tree, then the four partials meet in LDS.
static __device__ __forceinline__ float block_reduce(float v, float* sm) {
    v = WAVE_RED(v);
    const u32 lane = threadIdx.x & 63u, w = threadIdx.x >> 6;
    if (lane == 0) sm[w] = v;
    __syncthreads();
    v = COMB(COMB(sm[0], sm[1]), COMB(sm[2], sm[3]));
    __syncthreads();
    return v;
}
"""


def _ld4_define(nt: bool) -> str:
    """LD4(p): how a reduction reads 16 bytes -- streaming (nontemporal) for inputs far larger
    than the caches, ordinary otherwise."""
    return "\n#define LD4(p) ld4_stream(p)\n" if nt else "\n#define LD4(p) (*(p))\n"


def _red_defs(op: str) -> str:
    ident, comb, wred = _RED[op]
    return (f"#define IDENT {ident}\n#define COMB(a, b) {comb.format(a='(a)', b='(b)')}\n"
            f"#define WAVE_RED {wred}\n")


@cache
def reduce_full_kernel(op: str, vec: int, nt: bool = False) -> tuple[str, str, str]:
    """Stage kernel of the full reduction (cpu_kernel.py:150-177): block b folds the
    contiguous slice [b*chunk, (b+1)*chunk) of x (in units of `vec` floats) into one
    value, out[b] = value / divisor.  Contiguous slices (32 KiB per block, walked 16 KiB
    at a time with four independent accumulators) keep every block on its own DRAM
    pages; a grid-strided walk of the same data measured ~10 % slower.  The launcher runs
    it once over x and once more, with one block, over the partials; `divisor` is 1
    except in the last stage of a mean."""
    name = f"reduce_full_{op}_v{vec}{'nt' if nt else ''}"
    if vec == 4:
        loop = _ld4_define(nt) + r"""
    const u32 nv = n >> 2;
    const float4* __restrict__ x4 = reinterpret_cast<const float4*>(x);
    float a0 = IDENT, a1 = IDENT, a2 = IDENT, a3 = IDENT;
    const u32 end = min(nv, (blockIdx.x + 1u) * chunk);
    u32 v = blockIdx.x * chunk + threadIdx.x;
    for (; v + 768u < end; v += 1024u) {
        const float4 p = LD4(x4 + v), q = LD4(x4 + v + 256u), r = LD4(x4 + v + 512u), s = LD4(x4 + v + 768u);
        a0 = COMB(a0, COMB(COMB(p.x, p.y), COMB(p.z, p.w)));
        a1 = COMB(a1, COMB(COMB(q.x, q.y), COMB(q.z, q.w)));
        a2 = COMB(a2, COMB(COMB(r.x, r.y), COMB(r.z, r.w)));
        a3 = COMB(a3, COMB(COMB(s.x, s.y), COMB(s.z, s.w)));
    }
    for (; v < end; v += 256u) {
        const float4 p = LD4(x4 + v);
        a0 = COMB(a0, COMB(COMB(p.x, p.y), COMB(p.z, p.w)));
    }
    float acc = COMB(COMB(a0, a1), COMB(a2, a3));
    if (blockIdx.x == 0 && threadIdx.x < (n & 3u)) acc = COMB(acc, x[(nv << 2) + threadIdx.x]);
"""
    else:
        loop = r"""
    float a0 = IDENT, a1 = IDENT;
    const u32 end = min(n, (blockIdx.x + 1u) * chunk);
    u32 i = blockIdx.x * chunk + threadIdx.x;
    for (; i + 256u < end; i += 512u) { a0 = COMB(a0, x[i]); a1 = COMB(a1, x[i + 256u]); }
    if (i < end) a0 = COMB(a0, x[i]);
    float acc = COMB(a0, a1);
"""
    src = f"""{PRELUDE}{_red_defs(op)}{_BLOCK_REDUCE}
extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ x,
        float* __restrict__ out, u32 n, float divisor, u32 chunk) {{
    __shared__ float sm[4];
{loop}
    acc = block_reduce(acc, sm);
    if (threadIdx.x == 0) out[blockIdx.x] = acc / divisor;
}}
"""
    return src, name, _fmt("P", "P", "I", "f", "I")


@cache
def reduce_rows_kernel(op: str, vec: int, per_block: bool, nt: bool = False) -> tuple[str, str, str]:
    """out[r] = reduce over the contiguous row r of an (R, L) view, / divisor
    (the last-axis case of cpu_kernel.py:68-148).  Either one wavefront per row
    (four rows per 256-thread block) or, for long rows, one block per row."""
    name = f"reduce_rows_{op}_v{vec}_{'blk' if per_block else 'wav'}{'nt' if nt else ''}"
    T = "256u" if per_block else "64u"
    tid = "threadIdx.x" if per_block else "(threadIdx.x & 63u)"
    row = "blockIdx.x" if per_block else "(blockIdx.x * 4u + (threadIdx.x >> 6))"
    if vec == 4:
        loop = f"""
    const float4* __restrict__ p = reinterpret_cast<const float4*>(x + (u64)row * L);
    const u32 nv = L >> 2;
    float a0 = IDENT, a1 = IDENT;
    u32 v = {tid};
    for (; v + {T} < nv; v += 2u * {T}) {{
        const float4 s = LD4(p + v), t = LD4(p + v + {T});
        a0 = COMB(a0, COMB(COMB(s.x, s.y), COMB(s.z, s.w)));
        a1 = COMB(a1, COMB(COMB(t.x, t.y), COMB(t.z, t.w)));
    }}
    if (v < nv) {{ const float4 s = LD4(p + v); a0 = COMB(a0, COMB(COMB(s.x, s.y), COMB(s.z, s.w))); }}
    float acc = COMB(a0, a1);
"""
        loop = _ld4_define(nt) + loop
    else:
        loop = f"""
    const float* __restrict__ p = x + (u64)row * L;
    float acc = IDENT;
    for (u32 i = {tid}; i < L; i += {T}) acc = COMB(acc, p[i]);
"""
    if per_block:
        fin = """    acc = block_reduce(acc, sm);
    if (threadIdx.x == 0) out[row] = acc / divisor;"""
        guard = ""
    else:
        fin = """    acc = WAVE_RED(acc);
    if ((threadIdx.x & 63u) == 0) out[row] = acc / divisor;"""
        guard = "    if (row >= R) return;\n"
    src = f"""{PRELUDE}{_red_defs(op)}{_BLOCK_REDUCE}
extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ x,
        float* __restrict__ out, u32 R, u32 L, float divisor) {{
    __shared__ float sm[4];
    const u32 row = {row};
{guard}{loop}
{fin}
}}
"""
    return src, name, _fmt("P", "P", "I", "I", "f")


@cache
def reduce_cols_kernel(op: str, vec: int, ty: int = 4, nt: bool = False, TX: int = 64) -> tuple[str, str, str]:
    """out[o, c, i] = reduce over l in chunk c of x[o, l, i] for an (O, L, I) view, / divisor
    (the non-last-axis case of cpu_kernel.py:68-148, e.g. axis 0 of a matrix).

    The reference walks each column with stride I.  Here a 64 x ty block (ty = 4 or 16)
    owns 64*vec adjacent columns: lanes read consecutive addresses of one row (coalesced),
    the ty thread rows take every ty-th row of the chunk, and LDS joins them.  L is
    split into `chunks` so that tall, narrow inputs still fill the chip; the launcher
    reduces the (O, chunks, I) partials with a second call.  TX: lanes along a row (64, or 32 with
    twice the thread rows: half as many bytes of a row per block, which streams better beyond the caches)."""
    name = f"reduce_cols_{op}_v{vec}_y{ty}{'nt' if nt else ''}{f'_t{TX}' if TX != 64 else ''}"
    if vec == 4:
        defs = _ld4_define(nt) + """#define VT float4
#define LD(l) LD4(reinterpret_cast<const float4*>(xp + (u64)(l) * I))
#define ACC(a, t) { a.x = COMB(a.x, t.x); a.y = COMB(a.y, t.y); a.z = COMB(a.z, t.z); a.w = COMB(a.w, t.w); }
#define VINIT make_float4(IDENT, IDENT, IDENT, IDENT)
#define STORE(p, r) { r.x /= divisor; r.y /= divisor; r.z /= divisor; r.w /= divisor; reinterpret_cast<float4*>(p)[0] = r; }
"""
    else:
        defs = """#define VT float
#define LD(l) (xp[(u64)(l) * I])
#define ACC(a, t) { a = COMB(a, t); }
#define VINIT IDENT
#define STORE(p, r) { (p)[0] = r / divisor; }
"""
    src = f"""{PRELUDE}{_red_defs(op)}{defs}
extern "C" __global__ __launch_bounds__({TX * ty}) void {name}(const float* __restrict__ x,
        float* __restrict__ out, u32 L, u32 I, u32 chunk, float divisor) {{
    __shared__ VT sm[{ty}][{TX}];
    const u32 tx = threadIdx.x, ty = threadIdx.y, o = blockIdx.z;
    const u32 col = (blockIdx.x * {TX}u + tx) * {vec}u;
    const u32 l0 = blockIdx.y * chunk, l1 = min(L, l0 + chunk);
    VT a0 = VINIT, a1 = VINIT, a2 = VINIT, a3 = VINIT;
    if (col < I) {{
        const float* __restrict__ xp = x + (u64)o * L * I + col;
        u32 l = l0 + ty;
        for (; l + {3 * ty}u < l1; l += {4 * ty}u) {{
            const VT t0 = LD(l), t1 = LD(l + {ty}u), t2 = LD(l + {2 * ty}u), t3 = LD(l + {3 * ty}u);
            ACC(a0, t0) ACC(a1, t1) ACC(a2, t2) ACC(a3, t3)
        }}
        for (; l < l1; l += {ty}u) {{ const VT t0 = LD(l); ACC(a0, t0) }}
        ACC(a0, a1) ACC(a2, a3) ACC(a0, a2)
    }}
    sm[ty][tx] = a0;
    __syncthreads();
    if (ty == 0 && col < I) {{
        VT r = sm[0][tx];
        #pragma unroll
        for (int k = 1; k < {ty}; ++k) {{ const VT t = sm[k][tx]; ACC(r, t) }}
        STORE(out + ((u64)o * gridDim.y + blockIdx.y) * I + col, r)
    }}
}}
"""
    return src, name, _fmt("P", "P", "I", "I", "I", "f")


_ARGMAX_PAIR = r"""
// (value, index) pairs: the larger value wins, equal values keep the lower index, which is
// the index the reference's sequential `if (v > best)` scan ends with.  A scan starts from
// (-FLT_MAX, 0), so a row that never exceeds -FLT_MAX (all -inf, or NaN) answers 0, as there.
#define TAKE(bv, bi, ov, oi) if ((ov) > (bv) || ((ov) == (bv) && (oi) < (bi))) { bv = (ov); bi = (oi); }
static __device__ __forceinline__ void wave_argmax(float& best, u32& bi) {
    #pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(best, off, WAVE);
        const u32 oi = __shfl_xor(bi, off, WAVE);
        TAKE(best, bi, ov, oi)
    }
}
"""


@cache
def argmax_kernel(mode: str, vec: int = 1, unroll: int = 4, nt: bool = False, cap: int = 32) -> tuple[str, str, str]:
    """Index (as float) of the first maximum along L of an (O, L, I) view
    (cpu_kernel.py:459-517: strict '>', start value -FLT_MAX at index 0).
      rows_thread  I == 1, short rows, few of them: one thread per row
      rows_staged  I == 1, short rows (the (N, 10) class scores): 256 rows per block through LDS
      rows_wave    I == 1: one wavefront per row
      rows_block   I == 1, long rows (50304-wide logits): one block per row
      cols_part    I > 1: a 64 x 16 block owns 64 columns of one chunk of L; thread rows take
                   every 16th row, LDS joins them; writes the chunk's (value, index) per column,
                   or, when there is one chunk, the answer
      cols_fin     folds the chunks of cols_part in order
    vec = 4: 16-byte loads along the row (rows_staged / rows_wave / rows_block) or across four
    columns (cols_part); unroll: rows in flight per thread (cols_part); nt: streaming loads."""
    name = f"argmax_{mode}" + (f"_v{vec}" + ("nt" if nt and vec == 4 else "") if mode in ("rows_wave", "rows_block") else "")
    if mode == "rows_thread":
        src = f"""{PRELUDE}
extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ x,
        float* __restrict__ out, u32 R, u32 L) {{
    const u32 row = blockIdx.x * 256u + threadIdx.x;
    if (row >= R) return;
    const float* __restrict__ p = x + (u64)row * L;
    float best = NEG_FLT_MAX; u32 bi = 0;
    for (u32 i = 0; i < L; ++i) {{ const float v = p[i]; if (v > best) {{ best = v; bi = i; }} }}
    out[row] = (float)bi;
}}
"""
        return src, name, _fmt("P", "P", "I", "I")
    if mode == "rows_direct":
        # rows of an even number of floats up to cap, 8-byte aligned: every load of a row is issued before the first compare
        name = f"argmax_rows_direct_c{cap}"
        src = f"""{PRELUDE}
extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ x,
        float* __restrict__ out, u32 R, u32 L) {{
    const u32 row = blockIdx.x * 256u + threadIdx.x;
    if (row >= R) return;
    const float2* __restrict__ p = reinterpret_cast<const float2*>(x + (u64)row * L);
    float2 v[{cap // 2}];
    #pragma unroll
    for (u32 k = 0; k < {cap // 2}u; ++k) if (2u * k < L) v[k] = p[k];
    float best = NEG_FLT_MAX; u32 bi = 0;
    #pragma unroll
    for (u32 k = 0; k < {cap // 2}u; ++k) if (2u * k < L) {{
        if (v[k].x > best) {{ best = v[k].x; bi = 2u * k; }}
        if (v[k].y > best) {{ best = v[k].y; bi = 2u * k + 1u; }}
    }}
    out[row] = (float)bi;
}}
"""
        return src, name, _fmt("P", "P", "I", "I")
    if mode == "rows_staged":
        # rows of at most cap floats (sizes the LDS stage), loads of vec floats
        width = vec
        name = f"argmax_rows_staged_c{cap}_v{width}"
        if width == 4:
            fill = """
    u32 e = threadIdx.x * 4u, r = e / L, c = e % L;
    const u32 dq = 1024u / L, dr = 1024u % L;
    for (; e + 3u < n; e += 1024u) {
        const float4 v = ld4_stream(reinterpret_cast<const float4*>(p + e));
        u32 rr = r, cc = c;
        s[rr * Lp + cc] = v.x; if (++cc == L) { cc = 0; ++rr; }
        s[rr * Lp + cc] = v.y; if (++cc == L) { cc = 0; ++rr; }
        s[rr * Lp + cc] = v.z; if (++cc == L) { cc = 0; ++rr; }
        s[rr * Lp + cc] = v.w;
        c += dr; r += dq; if (c >= L) { c -= L; ++r; }
    }
    for (u32 t = (n & ~3u) + threadIdx.x; t < n; t += 256u) s[(t / L) * Lp + t % L] = p[t];"""
        else:
            fill = """
    u32 r = threadIdx.x / L, c = threadIdx.x % L;
    const u32 dq = 256u / L, dr = 256u % L;
    for (u32 e = threadIdx.x; e < n; e += 256u) {
        s[r * Lp + c] = p[e];
        c += dr; r += dq; if (c >= L) { c -= L; ++r; }
    }"""
        src = f"""{PRELUDE}
// 256 rows of L <= {cap} floats are one contiguous run: it is read with full-width coalesced
// loads into LDS (row pitch L | 1, so the per-row scans that follow hit distinct banks).
extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ x,
        float* __restrict__ out, u32 R, u32 L) {{
    __shared__ float s[256 * {cap | 1}];
    const u32 row0 = blockIdx.x * 256u;
    const u32 rows = min(256u, R - row0);
    const u32 n = rows * L, Lp = L | 1u;
    const float* __restrict__ p = x + (u64)row0 * L;
{fill}
    __syncthreads();
    if (threadIdx.x >= rows) return;
    const float* q = s + threadIdx.x * Lp;
    float best = NEG_FLT_MAX; u32 bi = 0;
    for (u32 i = 0; i < L; ++i) {{ const float v = q[i]; if (v > best) {{ best = v; bi = i; }} }}
    out[row0 + threadIdx.x] = (float)bi;
}}
"""
        return src, name, _fmt("P", "P", "I", "I")
    if mode in ("rows_wave", "rows_block"):
        blk = mode == "rows_block"
        T = "256u" if blk else "64u"
        tid = "threadIdx.x" if blk else "(threadIdx.x & 63u)"
        row = "blockIdx.x" if blk else "(blockIdx.x * 4u + (threadIdx.x >> 6))"
        if vec == 4:
            ld = "ld4_stream(p4 + " if nt else "*(p4 + "
            scan = f"""
    const float4* __restrict__ p4 = reinterpret_cast<const float4*>(p);
    #define STEP4(t, v) {{ const u32 i = (v) << 2; if (t.x > best) {{ best = t.x; bi = i; }} if (t.y > best) {{ best = t.y; bi = i + 1u; }} \\
                          if (t.z > best) {{ best = t.z; bi = i + 2u; }} if (t.w > best) {{ best = t.w; bi = i + 3u; }} }}
    u32 v = {tid};
    for (; v + 3u * {T} < (L >> 2); v += 4u * {T}) {{           // four loads in flight, compared in index order
        const float4 t0 = {ld}v), t1 = {ld}v + {T}), t2 = {ld}v + 2u * {T}), t3 = {ld}v + 3u * {T});
        STEP4(t0, v) STEP4(t1, v + {T}) STEP4(t2, v + 2u * {T}) STEP4(t3, v + 3u * {T})
    }}
    for (; v < (L >> 2); v += {T}) {{ const float4 t = {ld}v); STEP4(t, v) }}
    if ({tid} < (L & 3u)) {{ const u32 i = (L & ~3u) + {tid}; const float v = p[i]; TAKE(best, bi, v, i) }}
"""
        else:
            scan = f"""
    for (u32 i = {tid}; i < L; i += {T}) {{ const float v = p[i]; if (v > best) {{ best = v; bi = i; }} }}
"""
        if blk:
            fin = """    wave_argmax(best, bi);
    __shared__ float sv[4]; __shared__ u32 si[4];
    if ((threadIdx.x & 63u) == 0) { sv[threadIdx.x >> 6] = best; si[threadIdx.x >> 6] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        #pragma unroll
        for (int w = 1; w < 4; ++w) TAKE(best, bi, sv[w], si[w])
        out[row] = (float)bi;
    }"""
        else:
            fin = """    wave_argmax(best, bi);
    if ((threadIdx.x & 63u) == 0) out[row] = (float)bi;"""
        src = f"""{PRELUDE}{_ARGMAX_PAIR}
extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ x,
        float* __restrict__ out, u32 R, u32 L) {{
    const u32 row = {row};
    {'' if blk else 'if (row >= R) return;'}
    const float* __restrict__ p = x + (u64)row * L;
    float best = NEG_FLT_MAX; u32 bi = 0;
{scan}
{fin}
}}
"""
        return src, name, _fmt("P", "P", "I", "I")
    if mode == "cols_part":
        name += f"_v{vec}"
        if vec == 4:
            name += f"u{unroll}" + ("nt" if nt else "")
            ld = "ld4_stream(" if nt else "*("
            loads = "\n".join(f"            const float4 v{u} = {ld}reinterpret_cast<const float4*>(xp + (u64)(l + {16 * u}u) * I));"
                              for u in range(unroll))
            steps = " ".join(f"STEP(v{u}, l + {16 * u}u)" for u in range(unroll))
            scan = f"""
        #define STEP(v, l) {{ if (v.x > best[0]) {{ best[0] = v.x; bi[0] = (l); }} if (v.y > best[1]) {{ best[1] = v.y; bi[1] = (l); }} \\
                             if (v.z > best[2]) {{ best[2] = v.z; bi[2] = (l); }} if (v.w > best[3]) {{ best[3] = v.w; bi[3] = (l); }} }}
        u32 l = l0 + ty;
        for (; l + {16 * (unroll - 1)}u < l1; l += {16 * unroll}u) {{                  // {unroll} rows in flight, compared in row order
{loads}
            {steps}
        }}
        for (; l < l1; l += 16u) {{ const float4 v = {ld}reinterpret_cast<const float4*>(xp + (u64)l * I)); STEP(v, l) }}"""
        else:
            scan = """
        for (u32 l = l0 + ty; l < l1; l += 16u) { const float v = xp[(u64)l * I]; if (v > best[0]) { best[0] = v; bi[0] = l; } }"""
        src = f"""{PRELUDE}{_ARGMAX_PAIR}
#define VEC {vec}
extern "C" __global__ __launch_bounds__(1024) void {name}(const float* __restrict__ x,
        float* __restrict__ out, float* __restrict__ pv, u32* __restrict__ pi, u32 L, u32 I, u32 chunk, u32 final) {{
    __shared__ float sv[16][VEC][64]; __shared__ u32 si[16][VEC][64];     // [thread row][component][lane]: a wavefront's accesses fall on 64 consecutive words
    const u32 tx = threadIdx.x, ty = threadIdx.y, o = blockIdx.z;
    const u32 col = (blockIdx.x * 64u + tx) * VEC;
    const u32 l0 = blockIdx.y * chunk, l1 = min(L, l0 + chunk);
    float best[VEC]; u32 bi[VEC];
    #pragma unroll
    for (int c = 0; c < VEC; ++c) {{ best[c] = NEG_FLT_MAX; bi[c] = 0; }}
    if (col < I) {{
        const float* __restrict__ xp = x + (u64)o * L * I + col;{scan}
    }}
    #pragma unroll
    for (int c = 0; c < VEC; ++c) {{ sv[ty][c][tx] = best[c]; si[ty][c][tx] = bi[c]; }}
    __syncthreads();
    if (ty == 0 && col < I) {{
        #pragma unroll
        for (int c = 0; c < VEC; ++c) {{
            #pragma unroll
            for (int k = 1; k < 16; ++k) TAKE(best[c], bi[c], sv[k][c][tx], si[k][c][tx])
            if (final) out[(u64)o * I + col + c] = (float)bi[c];
            else {{ const u64 at = ((u64)o * gridDim.y + blockIdx.y) * I + col + c; pv[at] = best[c]; pi[at] = bi[c]; }}
        }}
    }}
}}
"""
        return src, name, _fmt("P", "P", "P", "P", "I", "I", "I", "I")
    assert mode == "cols_fin"
    src = f"""{PRELUDE}{_ARGMAX_PAIR}
// 64 columns x 16 chunk lanes per block: lane ty folds chunks ty, ty + 16, ..., LDS joins the lanes
extern "C" __global__ __launch_bounds__(1024) void {name}(const float* __restrict__ pv,
        const u32* __restrict__ pi, float* __restrict__ out, u32 O, u32 chunks, u32 I) {{
    __shared__ float sv[16][65]; __shared__ u32 si[16][65];
    const u32 tx = threadIdx.x, ty = threadIdx.y, o = blockIdx.y;
    const u32 col = blockIdx.x * 64u + tx;
    float best = NEG_FLT_MAX; u32 bi = 0;
    if (col < I)
        for (u32 c = ty; c < chunks; c += 16u) {{
            const u64 at = ((u64)o * chunks + c) * I + col;
            const float v = pv[at]; const u32 i = pi[at];
            TAKE(best, bi, v, i)
        }}
    sv[ty][tx] = best; si[ty][tx] = bi;
    __syncthreads();
    if (ty == 0 && col < I) {{
        #pragma unroll
        for (int k = 1; k < 16; ++k) TAKE(best, bi, sv[k][tx], si[k][tx])
        out[(u64)o * I + col] = (float)bi;
    }}
}}
"""
    return src, name, _fmt("P", "P", "P", "I", "I", "I")


# =====================================================================================
# permute
# =====================================================================================

@cache
def permute_gather_kernel(vec: int, nt: bool = False) -> tuple[str, str, str]:
    """out (contiguous, <=4-D, padded on the left) <- x read through permuted strides
    (cpu_kernel.py:179-215), for permutations that keep the innermost dim innermost:
    both sides are then contiguous along that dim and each thread moves `vec` floats.
    vec=4 needs the inner extent, every input stride and both bases to be multiples of 4."""
    nt = nt and vec == 4                                  # streaming form for tensors far larger than the caches
    name = f"permute_gather_v{vec}{'nt' if nt else ''}"
    if nt:
        move = ("{ const v4f t = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(x + off)); "
                "__builtin_nontemporal_store(t, reinterpret_cast<v4f*>(out) + i); }")
        scale = "const u32 c3 = (r % shape.d[3]) << 2; r /= shape.d[3];"
    elif vec == 4:
        move = ("reinterpret_cast<float4*>(out)[i] = "
                "reinterpret_cast<const float4*>(x + off)[0];")
        scale = "const u32 c3 = (r % shape.d[3]) << 2; r /= shape.d[3];"   # shape.d[3] is in float4 units
    else:
        move = "out[i] = x[off];"
        scale = "const u32 c3 = r % shape.d[3]; r /= shape.d[3];"
    src = f"""{PRELUDE}
struct Dims4 {{ u32 d[4]; }};
extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ x,
        float* __restrict__ out, u32 n, Dims4 shape, Dims4 st) {{
    const u32 i0 = blockIdx.x * 1024u + threadIdx.x;
    #pragma unroll
    for (int u = 0; u < 4; ++u) {{
        const u32 i = i0 + u * 256u;
        if (i < n) {{
            u32 r = i;
            {scale}
            const u32 c2 = r % shape.d[2]; r /= shape.d[2];
            const u32 c1 = r % shape.d[1];
            const u32 c0 = r / shape.d[1];
            const u64 off = (u64)c0 * st.d[0] + (u64)c1 * st.d[1] + (u64)c2 * st.d[2] + c3;
            {move}
        }}
    }}
}}
"""
    return src, name, _fmt("P", "P", "I", "4I", "4I")


@cache
def permute_tiled_kernel(vec: int = 1, swz: int = 0, tile: int = 64, nt: bool = False) -> tuple[str, str, str]:
    """Permutations that move another dim into the innermost position, e.g. (.., a, b) ->
    (.., b, a) or (B,T,h,d) -> (B,h,d,T).  Out dims are (p, q, t, b) after padding where
    b is the out-innermost dim and t is the out dim whose *input* stride is 1.  A tile of
    the (t, b) plane goes through LDS (rows padded by one float) so that reads run along t
    and writes along b, both coalesced; p and q only offset the tile.
    vec = 1: 32 x 32 tile, 4-byte accesses.  vec = 4: tile x tile (64 or 128), 16-byte loads
    along t and 16-byte stores along b; needs extents and strides that are multiples of 4 and
    16-byte aligned bases.
    swz = 1 walks the tiles of one block row diagonally: when the input's row pitch is a large
    power of two, the tiles that run at the same time otherwise read the same few memory
    channels.  nt: streaming loads and stores (planes far larger than the caches).
    The reference reads with the large stride directly (cpu_kernel.py:207-212)."""
    name = "permute_tiled" + ("_v4" if vec == 4 else "") + (f"_t{tile}" if tile != 64 else "") \
        + (f"_s{swz}" if swz else "") + ("nt" if nt else "")
    head = f"""{PRELUDE}
struct PArgs {{ u32 np, nq, nt, nb;        // extents: two carried dims, tile dims t and b
               u32 ip, iq, ib;            // input strides of p, q, b (t has input stride 1)
               u32 op, oq, ot; }};        // output strides of p, q, t (b has output stride 1)
"""
    if vec == 4:
        assert tile in (64, 128)
        lanes = tile // 4                 # threads across one tile row
        rows = 256 // lanes               # tile rows per pass of the block
        passes = tile // rows
        order = {0: """    const u32 bb = r % tb; r /= tb;
    const u32 bt = r % tt; r /= tt;""",
                 1: """    const u32 bb = r % tb; r /= tb;
    const u32 bt = (r % tt + bb) % tt; r /= tt;"""}[swz]
        load = "ld4_stream(reinterpret_cast<const float4*>(xi + (u64)b * a.ib + t))" if nt \
            else "*reinterpret_cast<const float4*>(xi + (u64)b * a.ib + t)"
        store = ("{ const v4f o = {tile[lb][lt], tile[lb + 1u][lt], tile[lb + 2u][lt], tile[lb + 3u][lt]};\n"
                 "              __builtin_nontemporal_store(o, reinterpret_cast<v4f*>(oo + (u64)t * a.ot + b)); }") if nt \
            else ("*reinterpret_cast<float4*>(oo + (u64)t * a.ot + b) =\n"
                  "                make_float4(tile[lb][lt], tile[lb + 1u][lt], tile[lb + 2u][lt], tile[lb + 3u][lt]);")
        src = head + f"""extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ x,
        float* __restrict__ out, PArgs a) {{
    __shared__ float tile[{tile}][{tile + 1}];          // [b][t]
    const u32 tb = (a.nb + {tile - 1}u) / {tile}u, tt = (a.nt + {tile - 1}u) / {tile}u;
    u32 r = blockIdx.x;
{order}
    const u32 q = r % a.nq, p = r / a.nq;
    const float* __restrict__ xi = x + (u64)p * a.ip + (u64)q * a.iq;
    float* __restrict__ oo = out + (u64)p * a.op + (u64)q * a.oq;
    const u32 c4 = threadIdx.x % {lanes}u, rw = threadIdx.x / {lanes}u;
    float4 v[{passes}];
    #pragma unroll
    for (u32 k = 0; k < {passes}u; ++k) {{              // every load in flight before the first LDS write
        const u32 t = bt * {tile}u + 4u * c4, b = bb * {tile}u + rw + {rows}u * k;
        v[k] = (t < a.nt && b < a.nb) ? {load}
                                      : make_float4(0.f, 0.f, 0.f, 0.f);
    }}
    #pragma unroll
    for (u32 k = 0; k < {passes}u; ++k) {{
        float* __restrict__ d = &tile[rw + {rows}u * k][4u * c4];
        d[0] = v[k].x; d[1] = v[k].y; d[2] = v[k].z; d[3] = v[k].w;
    }}
    __syncthreads();
    #pragma unroll
    for (u32 k = 0; k < {tile}u; k += {rows}u) {{
        const u32 t = bt * {tile}u + rw + k, b = bb * {tile}u + 4u * c4;
        if (t < a.nt && b < a.nb) {{
            const u32 lt = rw + k, lb = 4u * c4;
            {store}
        }}
    }}
}}
"""
        return src, name, _fmt("P", "P", "10I")
    src = head + f"""extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ x,
        float* __restrict__ out, PArgs a) {{
    __shared__ float tile[32][33];
    const u32 tb = (a.nb + 31u) >> 5, tt = (a.nt + 31u) >> 5;
    u32 r = blockIdx.x;
    const u32 bb = r % tb; r /= tb;
    const u32 bt = r % tt; r /= tt;
    const u32 q = r % a.nq, p = r / a.nq;
    const float* __restrict__ xi = x + (u64)p * a.ip + (u64)q * a.iq;
    float* __restrict__ oo = out + (u64)p * a.op + (u64)q * a.oq;
    const u32 tx = threadIdx.x & 31u, ty = threadIdx.x >> 5;
    #pragma unroll
    for (u32 k = 0; k < 32u; k += 8u) {{
        const u32 t = bt * 32u + tx, b = bb * 32u + ty + k;
        if (t < a.nt && b < a.nb) tile[ty + k][tx] = xi[(u64)b * a.ib + t];
    }}
    __syncthreads();
    #pragma unroll
    for (u32 k = 0; k < 32u; k += 8u) {{
        const u32 t = bt * 32u + ty + k, b = bb * 32u + tx;
        if (t < a.nt && b < a.nb) oo[(u64)t * a.ot + b] = tile[tx][ty + k];
    }}
}}
"""
    return src, name, _fmt("P", "P", "10I")


# =====================================================================================
# embedding, cross-entropy helpers, fused softmax
# =====================================================================================

@cache
def embedding_kernel() -> tuple[str, str, str]:
    """Gather: out[i, :] = x[(int)(idx[i] * W) + 0..W) (cpu_kernel.py:217-229; the
    offset is formed in float and truncated, exactly as there).  One wavefront per
    index; 16-byte moves when W and the offset allow it.  An index whose row does not lie
    inside the table's `total` floats (negative, or >= the row count) reads nothing: its
    output row is zeros (the reference reads whatever memory lies there)."""
    name = "embedding_gather"
    src = f"""{PRELUDE}
extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ x,
        const float* __restrict__ idx, float* __restrict__ out, u32 n_idx, u32 W, u32 aligned, u32 total) {{
    const u32 i = blockIdx.x * 4u + (threadIdx.x >> 6), lane = threadIdx.x & 63u;
    if (i >= n_idx) return;
    const int x_idx = (int)(idx[i] * (float)W);
    const float* __restrict__ src = x + (long long)x_idx;
    float* __restrict__ dst = out + (u64)i * W;
    if (x_idx < 0 || (u64)x_idx + W > (u64)total) {{
        for (u32 j = lane; j < W; j += 64u) dst[j] = 0.0f;
    }} else if (aligned && ((x_idx & 3) == 0)) {{
        for (u32 v = lane; v < (W >> 2); v += 64u)
            reinterpret_cast<float4*>(dst)[v] = reinterpret_cast<const float4*>(src)[v];
    }} else {{
        for (u32 j = lane; j < W; j += 64u) dst[j] = src[j];
    }}
}}
"""
    return src, name, _fmt("P", "P", "P", "I", "I", "I", "I")


@cache
def embedding_sum_kernel() -> tuple[str, str, str]:
    """out[i, :] = tok_table[idx[i]] + pos_table[pos[i % T]] for n = B * T positions: the token and position
    embeddings of a transformer's input and their sum (examples/gpt.py:96-98: two gathers and a broadcast add)
    in one launch.  Rows are looked up as embedding_kernel does it (offset (int)(id * W) formed in float, a row
    outside its table reads as zeros) and the sum is the one fp32 addition of the add kernel: same bits.
    One wavefront per position."""
    name = "embedding_sum"
    src = f"""{PRELUDE}
extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ tok_table,
        const float* __restrict__ pos_table, const float* __restrict__ idx, const float* __restrict__ pos,
        float* __restrict__ out, u32 n, u32 T, u32 W, u32 tok_total, u32 pos_total, u32 aligned) {{
    const u32 i = blockIdx.x * 4u + (threadIdx.x >> 6), lane = threadIdx.x & 63u;
    if (i >= n) return;
    const int ti = (int)(idx[i] * (float)W), pi = (int)(pos[i % T] * (float)W);
    const bool tok_ok = ti >= 0 && (u64)ti + W <= (u64)tok_total, pos_ok = pi >= 0 && (u64)pi + W <= (u64)pos_total;
    const float* __restrict__ a = tok_table + (long long)(tok_ok ? ti : 0);
    const float* __restrict__ b = pos_table + (long long)(pos_ok ? pi : 0);
    float* __restrict__ dst = out + (u64)i * W;
    if (aligned && tok_ok && pos_ok && ((ti | pi) & 3) == 0) {{
        for (u32 v = lane; v < (W >> 2); v += 64u) {{
            const float4 p = reinterpret_cast<const float4*>(a)[v], q = reinterpret_cast<const float4*>(b)[v];
            reinterpret_cast<float4*>(dst)[v] = make_float4(p.x + q.x, p.y + q.y, p.z + q.z, p.w + q.w);
        }}
    }} else {{
        for (u32 j = lane; j < W; j += 64u) dst[j] = (tok_ok ? a[j] : 0.0f) + (pos_ok ? b[j] : 0.0f);
    }}
}}
"""
    return src, name, _fmt("P", "P", "P", "P", "P", "I", "I", "I", "I", "I", "I")


@cache
def embedding_backward_kernel() -> tuple[str, str, str]:
    """Scatter-add: out[(int)idx[i], j] += g[i, j] into a zeroed (V, W) table
    (cpu_kernel.py:231-243).  The row index is formed in integers; the reference forms
    idx*W + j in float, which is the same number wherever that product is exact
    (below 2^24) and a wrong column above.  Hardware fp32 atomics, one wavefront per
    index row, so duplicate ids accumulate in an unspecified order.  Rows whose index is
    outside [0, V) are skipped."""
    name = "embedding_scatter_add"
    src = f"""{PRELUDE}
extern "C" __global__ __launch_bounds__(256) void {name}(float* __restrict__ out,
        const float* __restrict__ g, const float* __restrict__ idx, u32 n_idx, u32 W, u32 V) {{
    const u32 i = blockIdx.x * 4u + (threadIdx.x >> 6), lane = threadIdx.x & 63u;
    if (i >= n_idx) return;
    const int row = (int)idx[i];
    if ((u32)row >= V) return;
    float* __restrict__ dst = out + (long long)row * W;
    const float* __restrict__ src = g + (u64)i * W;
    for (u32 j = lane; j < W; j += 64u) unsafeAtomicAdd(dst + j, src[j]);
}}
"""
    return src, name, _fmt("P", "P", "P", "I", "I", "I")


EMB_SEGMENT = 512          # positions whose indices one round of the ordered scatter-add compares (eight ballots of 64)
EMB_ORDERED_MAX = 32768    # longest index list the ordered scatter-add takes: every position scans the whole list

WAVE_LDS_FENCE = r"""
// Values written to LDS by some lanes of a wavefront and read by others of the same wavefront
static __device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}
"""

_ORDERED_COMMON = WAVE_LDS_FENCE + f"""
#define EMB_SEG {EMB_SEGMENT}u
#define EMB_NK {EMB_SEGMENT // 64}
// Which positions of the segment [s0, s1) hold the id `my`: bit l of hit[k] stands for position
// s0 + 64 k + l.  All loads are issued before the first comparison; the masks are wave-uniform.
static __device__ __forceinline__ void segment_hits(const float* __restrict__ idx, int my, u32 s0, u32 s1,
                                                    u32 n, u32 lane, u64 (&hit)[EMB_NK]) {{
    float v[EMB_NK];
    #pragma unroll
    for (u32 k = 0; k < EMB_NK; ++k) v[k] = idx[min(s0 + 64u * k + lane, n - 1u)];
    #pragma unroll
    for (u32 k = 0; k < EMB_NK; ++k) hit[k] = __ballot(s0 + 64u * k + lane < s1 && (int)v[k] == my);
}}
// How many hits lie below local position li, and how many there are in all.
static __device__ __forceinline__ void hit_rank(const u64 (&hit)[EMB_NK], u32 li, u32& below, u32& total) {{
    below = 0; total = 0;
    #pragma unroll
    for (u32 k = 0; k < EMB_NK; ++k) {{
        total += (u32)__popcll(hit[k]);
        if (64u * k + 64u <= li) below += (u32)__popcll(hit[k]);
        else if (64u * k <= li) below += (u32)__popcll(hit[k] & ((1ull << (li - 64u * k)) - 1ull));
    }}
}}
"""


@cache
def embedding_backward_ordered_kernel(stage: str, vec: int = 1, nt: bool = False, ivec: int = 1) -> tuple[str, str, str]:
    """Deterministic scatter-add into a (V, W) table for up to EMB_ORDERED_MAX indices, without
    atomics on memory and without a zero-fill pass: three launches that together write every
    element of the table exactly once (cpu_kernel.py:231-243 zero-fills the table, then adds row i
    of the gradient to row idx[i]).

    The index list is cut into segments of EMB_SEGMENT positions.
      "mark"      a block per 64 consecutive table rows reads the index list once and collects, in
                  LDS, for each of its rows the set of segments the row's id occurs in; it writes
                  that set (a 64-bit mask, 0 = the id does not occur) to idsegs[row].  Every entry
                  of idsegs is written, so nothing needs clearing first.
      "segments"  two kinds of blocks share the grid.
         sum blocks: one wavefront per position i.  From the 512 indices of its segment (eight
           ballots) it learns r, how many earlier positions of the segment hold the same id, and
           m, how many hold it in all, and lists them in LDS.  The id's m wavefronts in the segment
           split the row's columns into m slices; the r-th adds, for its slice, the gradient rows
           of all m positions in index order starting from 0 -- the order of the reference's loop
           -- so a hot id costs its wavefronts no more than a rare one.  The (row, column) items of
           a slice are spread over all 64 lanes so that every load of a pass is in flight at once,
           meet in LDS, and each column is added in row order.  If idsegs says the id occurs in no
           other segment the sum is the final table row; otherwise it goes to partial[first
           position of the id in the segment], and that first position records the set of segments
           in segmask (0 for every other position), looks up g, the id's first position of all (one
           more round of ballots over the id's earliest segment), and enters itself in the list of
           the id's first positions that is kept at g: firsts[g][rank of its segment], gfirst[i] = g.
         zero blocks: each owns 64 consecutive table rows and writes zeros to those whose idsegs
           entry is 0.  They are spread evenly among the sum blocks, so that the stream of zeros
           (bandwidth-bound) and the sums (latency-bound) run side by side.
      "merge"     the first positions of an id that spans segments (segmask != 0) split the columns
                  again and add the id's partial rows in segment order, starting from the first.
    Every table row is written once: by a zero block, by the sum wavefronts of its only segment, or
    by the merge; the three sets are disjoint, so nothing races inside a launch.  An id confined to
    one segment has exactly the bits of the sequential reference loop; one that spans segments
    differs from it only in where the parentheses fall, and every run gives the same bits.  Ids
    outside [0, V) take no part.  vec = 4 moves rows as float4 (W % 4 == 0, 16-byte aligned bases);
    nt writes the zeros with nontemporal stores (tables far larger than the caches); ivec = 4 lets
    "mark" read the index list 16 bytes at a time (a 16-byte aligned list)."""
    assert stage in ("mark", "segments", "merge")
    name = (f"embedding_scatter_{stage}" + (f"_i{ivec}" if stage == "mark" else
            f"_v{vec}{'nt' if (nt and stage == 'segments' and vec == 4) else ''}"))
    VT = "float4" if vec == 4 else "float"
    zero = "make_float4(0.f, 0.f, 0.f, 0.f)" if vec == 4 else "0.0f"
    add = ("acc.x += t.x; acc.y += t.y; acc.z += t.z; acc.w += t.w;" if vec == 4 else "acc += t;")
    add_ = add.replace("t.", "t_.").replace("+= t;", "+= t_;")
    zstore = ("{ const v4f z = {0.f, 0.f, 0.f, 0.f}; __builtin_nontemporal_store(z, reinterpret_cast<v4f*>(zrow) + c); }"
              if (nt and vec == 4) else f"zrow[c] = {zero};")
    if ivec == 4:
        # positions 4 * item .. 4 * item + 3 per thread; an item that sticks out past n is judged value by value
        # eight items per thread and round: their loads are all issued before the first comparison
        mscan = """    for (u32 t0 = threadIdx.x; 4u * t0 < n; t0 += 2048u) {
        float4 q[8];
        #pragma unroll
        for (u32 u = 0; u < 8u; ++u) { const u32 t = t0 + 256u * u; if (4u * t + 3u < n) q[u] = reinterpret_cast<const float4*>(idx)[t]; }
        #pragma unroll
        for (u32 u = 0; u < 8u; ++u) {
            const u32 t = t0 + 256u * u;
            if (4u * t + 3u < n) { MARK(q[u].x, 4u * t) MARK(q[u].y, 4u * t + 1u) MARK(q[u].z, 4u * t + 2u) MARK(q[u].w, 4u * t + 3u) }
            else for (u32 p = 4u * t; p < n; ++p) MARK(idx[p], p)
        }
    }"""
    else:
        mscan = """    for (u32 t = threadIdx.x; t < n; t += 256u) MARK(idx[t], t)"""
    if stage == "mark":
        body = f"""
extern "C" __global__ __launch_bounds__(256) void {name}(u64* __restrict__ idsegs,
        const float* __restrict__ idx, u32 n, u32 V) {{
    __shared__ u32 lo[64], hi[64];                              // per row of this block: the segments its id occurs in
    const u32 v0 = blockIdx.x * 64u;
    if (threadIdx.x < 64u) {{ lo[threadIdx.x] = 0u; hi[threadIdx.x] = 0u; }}
    __syncthreads();
#define MARK(val, pos) {{ const int id = (int)(val); if (id >= (int)v0 && id < (int)v0 + 64) {{ const u32 sg = (pos) / EMB_SEG; \\
        atomicOr(sg < 32u ? &lo[id - (int)v0] : &hi[id - (int)v0], 1u << (sg & 31u)); }} }}
{mscan}
    __syncthreads();
    if (threadIdx.x < 64u && v0 + threadIdx.x < V) idsegs[v0 + threadIdx.x] = (u64)lo[threadIdx.x] | ((u64)hi[threadIdx.x] << 32);
}}
"""
        return f"{PRELUDE}{_ORDERED_COMMON}{body}", name, _fmt("P", "P", "I", "I")
    if stage == "segments":
        body = f"""
extern "C" __global__ __launch_bounds__(256) void {name}(float* __restrict__ out,
        float* __restrict__ partial, u64* __restrict__ segmask, u32* __restrict__ firsts, u32* __restrict__ gfirst,
        const u64* __restrict__ idsegs, const float* __restrict__ g, const float* __restrict__ idx, u32 n, u32 W, u32 V,
        u32 n_zero_blocks, u32 every) {{
    __shared__ u32 lists[4][{EMB_SEGMENT}];
    __shared__ {VT} stage[4][{EMB_SEGMENT}];
    const u32 w = threadIdx.x >> 6, lane = threadIdx.x & 63u;
    const u32 Wv = W / {vec}u;
    // every `every`-th block is a zero block until all n_zero_blocks of them are placed
    const u32 grp = blockIdx.x / every;
    if (blockIdx.x % every == every - 1u && grp < n_zero_blocks) {{
        // ---- a zero block: 64 table rows, zeros for those no index names
        const u32 v0 = grp * 64u;
        const u32 rows = min(64u, V - v0);
        // which of the rows some index names, read by every wavefront in one go (sixteen reads one after the other, each
        // deciding the next row's fate, would make the stream of zeros wait for sixteen round trips to memory)
        const u64 named = __ballot(lane < rows ? idsegs[v0 + lane] != 0ull : true);
        for (u32 r = w; r < rows; r += 4u) {{                     // a wavefront per row, rows four apart
            if ((named >> r) & 1ull) continue;                  // some index names this row: its sum is written instead
            {VT}* __restrict__ zrow = reinterpret_cast<{VT}*>(out + (u64)(v0 + r) * W);
            for (u32 c = lane; c < Wv; c += 64u) {zstore}
        }}
        return;
    }}
    // ---- a sum block: one wavefront per position
    const u32 i = (blockIdx.x - min(n_zero_blocks, grp)) * 4u + w;
    if (i >= n) return;
    const int my = (int)idx[i];
    const u32 seg = i / EMB_SEG, s0 = seg * EMB_SEG, s1 = min(n, s0 + EMB_SEG);
    u64 hit[EMB_NK];
    segment_hits(idx, my, s0, s1, n, lane, hit);                // (its loads do not wait for `my`)
    if ((u32)my >= V) {{ if (lane == 0u) segmask[i] = 0ull; return; }}     // wave-uniform: the whole wavefront leaves
    u32 r, m;                                                   // this position is the r-th of the id's m in the segment
    hit_rank(hit, i - s0, r, m);
    u32* __restrict__ list = lists[w];                          // the id's positions in the segment, ascending
    if (m == 1u) {{
        if (lane == 0u) list[0] = i;
    }} else {{
        u32 at = 0;
        #pragma unroll
        for (u32 k = 0; k < EMB_NK; ++k) {{
            if ((hit[k] >> lane) & 1ull) list[at + (u32)__popcll(hit[k] & ((1ull << lane) - 1ull))] = s0 + 64u * k + lane;
            at += (u32)__popcll(hit[k]);
        }}
    }}
    const u64 segs = idsegs[my];                                // the segments the id occurs in (this one among them)
    wave_lds_fence();
    const bool other = segs != (1ull << seg);
    u64 mine = 0ull;                                            // what segmask[i] will hold
    if (r == 0u && other) {{                                     // the merge adds the partial rows of these first positions
        const u32 NS = (n + EMB_SEG - 1u) / EMB_SEG;
        const u32 tmin = (u32)__builtin_ctzll(segs);            // the id's earliest segment
        u32 gf = i;                                             // the id's first position of all: this one, in that segment
        if (tmin != seg) {{
            const u32 t0 = tmin * EMB_SEG;
            u64 h2[EMB_NK];
            segment_hits(idx, my, t0, min(n, t0 + EMB_SEG), n, lane, h2);
            gf = 0xFFFFFFFFu;
            #pragma unroll
            for (u32 j = EMB_NK; j-- > 0u;) if (h2[j]) gf = t0 + 64u * j + (u32)__builtin_ctzll(h2[j]);
        }}
        if (gf < n) {{                                           // (the mark launch saw the id there, so it is found)
            mine = segs;
            const u32 k = (u32)__popcll(segs & ((1ull << seg) - 1ull));        // this segment's rank among the id's
            if (lane == 0u) {{ firsts[(u64)gf * NS + k] = i; gfirst[i] = gf; }}
        }}
    }}
    if (lane == 0u) segmask[i] = mine;
    {VT}* __restrict__ dst = reinterpret_cast<{VT}*>(other ? partial + (u64)list[0] * W : out + (u64)my * W);
    const u32 c0 = r * Wv / m, c1 = (r + 1u) * Wv / m;        /* r < 512 and Wv < 2^22: no overflow */      // this wavefront's slice of the columns
    // The (row, column) items of the slice are spread over all 64 lanes, so every load of a pass
    // is in flight at once whatever m is; they meet in LDS, where each column is added in row order.
    {VT}* __restrict__ st = stage[w];
    const u32 cw = max(1u, EMB_SEG / m);                        // columns per pass: m * cw <= EMB_SEG items
    for (u32 cs = c0; cs < c1; cs += cw) {{
        const u32 cwn = min(cw, c1 - cs), items = m * cwn;
        for (u32 t0 = 0; t0 < items; t0 += 256u) {{
            {VT} v[4];
            #pragma unroll
            for (u32 u = 0; u < 4u; ++u) {{                     // loads past the end repeat the last item
                const u32 t = min(t0 + 64u * u + lane, items - 1u), q = t / cwn, cl = t - q * cwn;
                v[u] = reinterpret_cast<const {VT}*>(g + (u64)list[q] * W)[cs + cl];
            }}
            #pragma unroll
            for (u32 u = 0; u < 4u; ++u) {{
                const u32 t = t0 + 64u * u + lane;
                if (t < items) {{
                    if (m == 1u) {{ {VT} acc = {zero}; const {VT} t_ = v[u]; {add_} dst[cs + t] = acc; }}     // a single row: 0 + row, no staging
                    else st[t] = v[u];
                }}
            }}
        }}
        if (m == 1u) continue;
        wave_lds_fence();
        for (u32 cl = lane; cl < cwn; cl += 64u) {{
            {VT} acc = {zero};
            #pragma unroll 4
            for (u32 q = 0; q < m; ++q) {{ const {VT} t = st[q * cwn + cl]; {add} }}
            dst[cs + cl] = acc;
        }}
        wave_lds_fence();                                       // the next pass overwrites the stage
    }}
}}
"""
        fmt = _fmt("P", "P", "P", "P", "P", "P", "P", "P", "I", "I", "I", "I", "I")
    else:
        body = f"""
extern "C" __global__ __launch_bounds__(256) void {name}(float* __restrict__ out,
        const float* __restrict__ partial, const u64* __restrict__ segmask, const u32* __restrict__ firsts,
        const u32* __restrict__ gfirst, const float* __restrict__ idx, u32 n, u32 W, u32 V) {{
    const u32 w = threadIdx.x >> 6, lane = threadIdx.x & 63u;
    const u32 i = blockIdx.x * 4u + w;                          // one wavefront per position
    if (i >= n) return;
    const u64 segs = segmask[i];
    const float mine = idx[i];                                  // (read along with the mask: one trip to memory, not three)
    const u32 gf = gfirst[i];                                   // (a position only where the mask is set; unused elsewhere)
    if (segs == 0ull) return;                                   // only the first positions of an id that spans segments work
    const int my = (int)mine;
    const u32 m = (u32)__popcll(segs);
    const u32 r = (u32)__popcll(segs & ((1ull << (i / EMB_SEG)) - 1ull));           // this segment's rank among them
    // the id's first position in each of its segments, in segment order: each of them entered itself in the
    // list kept at the id's first position of all
    const u32* __restrict__ list = firsts + (u64)gf * ((n + EMB_SEG - 1u) / EMB_SEG);
    const u32 Wv = W / {vec}u;
    {VT}* __restrict__ dst = reinterpret_cast<{VT}*>(out + (u64)my * W);
    const u32 c0 = r * Wv / m, c1 = (r + 1u) * Wv / m;        /* r < 512 and Wv < 2^22: no overflow */      // the first positions split the columns
    for (u32 c = c0 + lane; c < c1; c += 64u) {{
        {VT} acc = reinterpret_cast<const {VT}*>(partial + (u64)list[0] * W)[c];
        #pragma unroll 8
        for (u32 q = 1; q < m; ++q) {{ const {VT} t = reinterpret_cast<const {VT}*>(partial + (u64)list[q] * W)[c]; {add} }}
        dst[c] = acc;
    }}
}}
"""
        fmt = _fmt("P", "P", "P", "P", "P", "P", "I", "I", "I")
    return f"{PRELUDE}{_ORDERED_COMMON}{body}", name, fmt


EMB_SMALL_MAX_N = 4096         # longest index list of the one-launch scatter-add: every row's wavefront reads all of it
EMB_SMALL_MAX_WAVES = 4096     # (table rows) x (column chunks) it is used for: beyond that the three-launch form has more to offer


@cache
def embedding_backward_small_kernel(vec: int = 1) -> tuple[str, str, str]:
    """Scatter-add into a small (V, W) table in one launch, in exactly the order of the reference's loop
    (cpu_kernel.py:231-243: zero the table, then out[idx[i]] += g[i] for i = 0, 1, ...).
    One wavefront per (table row, chunk of 64 * vec columns).  It reads the index list segment by segment
    (512 positions, eight ballots), lists the positions that name its row in LDS, and adds their gradient
    rows in index order, eight loads in flight; a row nobody names is written as zeros.  Every table element
    is written once, nothing is zero-filled first, no atomics: the bits are those of the sequential loop
    for every id, however its positions are spread.  Ids outside [0, V) take no part."""
    name = f"embedding_scatter_small_v{vec}"
    VT = "float4" if vec == 4 else "float"
    zero = "make_float4(0.f, 0.f, 0.f, 0.f)" if vec == 4 else "0.0f"
    add = ("acc.x += t[u].x; acc.y += t[u].y; acc.z += t[u].z; acc.w += t[u].w;" if vec == 4 else "acc += t[u];")
    body = f"""
extern "C" __global__ __launch_bounds__(256) void {name}(float* __restrict__ out, const float* __restrict__ g,
        const float* __restrict__ idx, u32 n, u32 W, u32 V, u32 chunks) {{
    __shared__ u32 lists[4][{EMB_SEGMENT}];
    const u32 w = threadIdx.x >> 6, lane = threadIdx.x & 63u;
    const u32 id = blockIdx.x * 4u + w;
    const u32 v = id / chunks;
    if (v >= V) return;
    const u32 Wv = W / {vec}u;
    const u32 c = (id - v * chunks) * 64u + lane;               // this lane's column item
    const bool live = c < Wv;
    u32* __restrict__ list = lists[w];
    {VT} acc = {zero};
    for (u32 s0 = 0; s0 < n; s0 += EMB_SEG) {{
        u64 hit[EMB_NK];
        segment_hits(idx, (int)v, s0, min(n, s0 + EMB_SEG), n, lane, hit);
        u32 m = 0;
        #pragma unroll
        for (u32 k = 0; k < EMB_NK; ++k) {{
            if ((hit[k] >> lane) & 1ull) list[m + (u32)__popcll(hit[k] & ((1ull << lane) - 1ull))] = s0 + 64u * k + lane;
            m += (u32)__popcll(hit[k]);
        }}
        if (m == 0u) continue;                                  // (wave-uniform)
        wave_lds_fence();
        for (u32 q0 = 0; q0 < m; q0 += 8u) {{
            {VT} t[8];
            #pragma unroll
            for (u32 u = 0; u < 8u; ++u)                        // loads past the end repeat the last row
                t[u] = live ? reinterpret_cast<const {VT}*>(g + (u64)list[min(q0 + u, m - 1u)] * W)[c] : {zero};
            #pragma unroll
            for (u32 u = 0; u < 8u; ++u) if (q0 + u < m) {{ {add} }}
        }}
        wave_lds_fence();                                       // the next segment overwrites the list
    }}
    if (live) reinterpret_cast<{VT}*>(out + (u64)v * W)[c] = acc;
}}
"""
    return f"{PRELUDE}{_ORDERED_COMMON}{body}", name, _fmt("P", "P", "P", "I", "I", "I", "I")


@cache
def ce_kernel(backward: bool) -> tuple[str, str, str]:
    """ce_forward: out[i] = x[(int)target[i] + stride0*i]; ce_backward: that element -= 1,
    in place (cpu_kernel.py:430-457).  A target outside [0, cols) picks 0 and subtracts nothing."""
    if backward:
        name = "ce_backward"
        src = f"""{PRELUDE}
extern "C" __global__ __launch_bounds__(256) void {name}(float* x, const float* __restrict__ target,
        u32 rows, u32 stride0, u32 cols) {{
    const u32 i = blockIdx.x * 256u + threadIdx.x;
    if (i >= rows) return;
    const int t = (int)target[i];
    if ((u32)t < cols) x[(long long)t + (u64)stride0 * i] -= 1.0f;
}}
"""
        return src, name, _fmt("P", "P", "I", "I", "I")
    name = "ce_forward"
    src = f"""{PRELUDE}
extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ x,
        const float* __restrict__ target, float* __restrict__ out, u32 rows, u32 stride0, u32 cols) {{
    const u32 i = blockIdx.x * 256u + threadIdx.x;
    if (i >= rows) return;
    const int t = (int)target[i];
    out[i] = (u32)t < cols ? x[(long long)t + (u64)stride0 * i] : 0.0f;
}}
"""
    return src, name, _fmt("P", "P", "P", "I", "I", "I")


def _row_block_reduce(NW: int) -> str:
    """block_max / block_sum over the NW wavefronts of a block that owns one row: the per-wave
    results meet in LDS and are combined in wave order by every thread."""
    return f"""
static __device__ __forceinline__ float block_max(float v, float* sm) {{
    v = wave_max(v);
    if ((threadIdx.x & 63u) == 0) sm[threadIdx.x >> 6] = v;
    __syncthreads();
    v = sm[0];
    #pragma unroll
    for (int w = 1; w < {NW}; ++w) v = fmaxf(v, sm[w]);
    __syncthreads();
    return v;
}}
static __device__ __forceinline__ float block_sum(float v, float* sm) {{
    v = wave_sum(v);
    if ((threadIdx.x & 63u) == 0) sm[threadIdx.x >> 6] = v;
    __syncthreads();
    v = sm[0];
    #pragma unroll
    for (int w = 1; w < {NW}; ++w) v += sm[w];
    __syncthreads();
    return v;
}}
"""


@cache
def softmax_rows_kernel(log: bool, vec: int, per_block: bool, nval: int = 0, gather: bool = False,
                        threads: int = 256, nt: bool = False, masked: bool = False) -> tuple[str, str, str]:
    """Row softmax / log-softmax over the contiguous last axis of an (R, L) view, replacing
    the reference's five kernels and four temporaries (tensor.py:634-669).  Same formula:
    e = exp(x - max); e / sum(e)   (or (x - max) - log(sum)).

    One wavefront per row, or one block of `threads` threads per long row.  nval > 0 is the
    register-resident form: each thread keeps its nval float4 (or float) items of the row
    in registers, so the row is read from HBM once and written once (8 B per element, the
    algorithmic minimum); rows of 50304 floats fit in 50 float4 per thread of a block.
    nval = 0 streams the row three times (for rows longer than registers hold).
    gather (log-softmax only): also writes picked[row] = out[row, (int)target[row]], the
    ce_forward gather of cpu_kernel.py:430-441, fused.
    masked (register-resident forms): the row is x * scale with -inf where mask > 0, the
    attention chain `(att * scale).masked_fill(mask, -inf).softmax()` of examples/gpt.py:51-54
    in one pass; the mask has `mrows` rows of L and row r of x uses mask row r % mrows.
    masked = "causal" (16-byte items): the mask is known to be 1 exactly where column > r % mrows (what
    ops.causal_mask builds), so it is computed from the indices and never read: same values, and the
    pass over the mask through the L2 -- as many bytes as the output -- disappears."""
    if not per_block:
        threads = 256
    causal = masked == "causal"                           # the mask is "column > row % mrows": computed, not read
    masked = bool(masked)
    assert not masked or (nval and not gather)
    assert not causal or vec == 4
    nt = nt and bool(nval) and vec == 4                   # streaming loads/stores: register-resident float4 form only
    name = (f"{'log_' if log else ''}softmax_rows_v{vec}_{f'blk{threads}' if per_block else 'wav'}"
            f"{f'_r{nval}' if nval else ''}{'_g' if gather else ''}{'_c' if causal else '_m' if masked else ''}{'nt' if nt else ''}")
    T = f"{threads}u" if per_block else "64u"
    NW = threads // 64
    tid = "threadIdx.x" if per_block else "(threadIdx.x & 63u)"
    row = "blockIdx.x" if per_block else "(blockIdx.x * 4u + (threadIdx.x >> 6))"
    red_max = "block_max(m, sm)" if per_block else "wave_max(m)"
    red_sum = "block_sum(s, sm)" if per_block else "wave_sum(s)"

    # Register-resident softmax (not log-softmax): each exp(x - m) is computed once, kept in the register
    # that held x, summed, and divided by the sum afterwards -- the values and the order of the
    # five-kernel composition (the exp kernel's output is what its sum and its division read).
    keep = bool(nval) and not log

    def outexpr(v: str) -> str:
        return f"(({v}) - m) - ls" if log else (f"({v}) / s" if keep else f"expf(({v}) - m) / s")
    comps = ("x", "y", "z", "w")
    keep_exp4 = "".join(f"        v[k].{c} = expf(v[k].{c} - m);\n" for c in comps) if keep else ""
    keep_exp1 = "v[k] = expf(v[k] - m); " if keep else ""
    mask4 = mask1 = ""
    if masked:
        sel4 = " ".join(f"v[k].{c} = (mb[k] & {1 << j}u) ? -__builtin_inff() : v[k].{c} * scale;" for j, c in enumerate(comps))
        ldx = "ld4_stream(p + c)" if nt else "p[c]"
        # the mask is read first (a few rows, cache resident); items that are masked in all four
        # lanes are never loaded, which halves the reads of a causal mask
        if causal:
            mask_bits = ("    const u32 last = row % mrows;                             // the last column this row may look at\n",
                         "mb[k] = (4u * c > last ? 1u : 0u) | (4u * c + 1u > last ? 2u : 0u) | (4u * c + 2u > last ? 4u : 0u) | (4u * c + 3u > last ? 8u : 0u);")
        else:
            mask_bits = ("    const float4* __restrict__ pm = reinterpret_cast<const float4*>(mask + (u64)(row % mrows) * L);\n",
                         "const float4 mk = pm[c]; mb[k] = (mk.x > 0.0f ? 1u : 0u) | (mk.y > 0.0f ? 2u : 0u) | (mk.z > 0.0f ? 4u : 0u) | (mk.w > 0.0f ? 8u : 0u);")
        mask4 = f"""{mask_bits[0]}    u32 mb[{nval}];
    #pragma unroll
    for (u32 k = 0; k < {nval}u; ++k) {{
        const u32 c = {tid} + k * {T};
        mb[k] = 15u;
        if (c < nv) {{ {mask_bits[1]} }}
    }}
    #pragma unroll
    for (u32 k = 0; k < {nval}u; ++k) {{ const u32 c = {tid} + k * {T}; v[k] = make_float4(0.f, 0.f, 0.f, 0.f); if (mb[k] != 15u) v[k] = {ldx}; }}
    #pragma unroll
    for (u32 k = 0; k < {nval}u; ++k) {{ {sel4} }}
"""
        mask1 = f"""    const float* __restrict__ pm = mask + (u64)(row % mrows) * L;
    #pragma unroll
    for (u32 k = 0; k < {nval}u; ++k) {{ const u32 c = {tid} + k * {T}; if (c < L) v[k] = pm[c] > 0.0f ? -__builtin_inff() : v[k] * scale; }}
"""
    load4 = mask4 if masked else (f"    #pragma unroll\n    for (u32 k = 0; k < {nval}u; ++k) {{ const u32 c = {tid} + k * {T}; "
                                  f"if (c < nv) v[k] = {'ld4_stream(p + c)' if nt else 'p[c]'}; }}\n")
    if nval and vec == 4:
        # with a mask, items masked in all four lanes (mb[k] == 15, also set beyond the row's end) take no
        # part in the max or the sum and are written as zeros, which is what exp(-inf - m) / s gives
        live = "mb[k] != 15u" if masked else f"{tid} + k * {T} < nv"
        zero_dead = "            if (mb[k] == 15u) o = make_float4(0.f, 0.f, 0.f, 0.f); else {\n" if masked else ""
        close_dead = "            }\n" if masked else ""
        body = f"""
    const float4* __restrict__ p = reinterpret_cast<const float4*>(x + (u64)row * L);
    float4* __restrict__ q = reinterpret_cast<float4*>(out + (u64)row * L);
    const u32 nv = L >> 2;
    float4 v[{nval}];
{load4}    float m = NEG_FLT_MAX;
    #pragma unroll
    for (u32 k = 0; k < {nval}u; ++k) if ({live})
        m = fmaxf(fmaxf(m, fmaxf(v[k].x, v[k].y)), fmaxf(v[k].z, v[k].w));
    m = {red_max};
    float s = 0.0f;
    #pragma unroll
    for (u32 k = 0; k < {nval}u; ++k) if ({live}) {{
{keep_exp4}        s += (E(v[k].x) + E(v[k].y)) + (E(v[k].z) + E(v[k].w));
    }}
    s = {red_sum};
    const float ls = logf(s); (void)ls;
    #pragma unroll
    for (u32 k = 0; k < {nval}u; ++k) {{
        const u32 c = {tid} + k * {T};
        if (c < nv) {{
            float4 o;
{zero_dead}{''.join(f"            o.{c} = {outexpr(f'v[k].{c}')};{chr(10)}" for c in comps)}{close_dead}            {'{ const v4f ov = {o.x, o.y, o.z, o.w}; __builtin_nontemporal_store(ov, reinterpret_cast<v4f*>(q) + c); }' if nt else 'q[c] = o;'}
        }}
    }}
"""
    elif nval:
        body = f"""
    const float* __restrict__ p = x + (u64)row * L;
    float* __restrict__ q = out + (u64)row * L;
    float v[{nval}];
    #pragma unroll
    for (u32 k = 0; k < {nval}u; ++k) {{ const u32 c = {tid} + k * {T}; if (c < L) v[k] = p[c]; }}
{mask1}    float m = NEG_FLT_MAX;
    #pragma unroll
    for (u32 k = 0; k < {nval}u; ++k) if ({tid} + k * {T} < L) m = fmaxf(m, v[k]);
    m = {red_max};
    float s = 0.0f;
    #pragma unroll
    for (u32 k = 0; k < {nval}u; ++k) if ({tid} + k * {T} < L) {{ {keep_exp1}s += E(v[k]); }}
    s = {red_sum};
    const float ls = logf(s); (void)ls;
    #pragma unroll
    for (u32 k = 0; k < {nval}u; ++k) {{ const u32 c = {tid} + k * {T}; if (c < L) q[c] = {outexpr('v[k]')}; }}
"""
    elif vec == 4:
        body = f"""
    const float4* __restrict__ p = reinterpret_cast<const float4*>(x + (u64)row * L);
    float4* __restrict__ q = reinterpret_cast<float4*>(out + (u64)row * L);
    const u32 nv = L >> 2;
    float m = NEG_FLT_MAX;
    for (u32 c = {tid}; c < nv; c += {T}) {{ const float4 t = p[c]; m = fmaxf(fmaxf(m, fmaxf(t.x, t.y)), fmaxf(t.z, t.w)); }}
    m = {red_max};
    float s = 0.0f;
    for (u32 c = {tid}; c < nv; c += {T}) {{ const float4 t = p[c]; s += (expf(t.x - m) + expf(t.y - m)) + (expf(t.z - m) + expf(t.w - m)); }}
    s = {red_sum};
    const float ls = logf(s); (void)ls;
    for (u32 c = {tid}; c < nv; c += {T}) {{
        const float4 t = p[c]; float4 o;
{''.join(f"        o.{c} = {outexpr(f't.{c}')};{chr(10)}" for c in comps)}        q[c] = o;
    }}
"""
    else:
        body = f"""
    const float* __restrict__ p = x + (u64)row * L;
    float* __restrict__ q = out + (u64)row * L;
    float m = NEG_FLT_MAX;
    for (u32 c = {tid}; c < L; c += {T}) m = fmaxf(m, p[c]);
    m = {red_max};
    float s = 0.0f;
    for (u32 c = {tid}; c < L; c += {T}) s += expf(p[c] - m);
    s = {red_sum};
    const float ls = logf(s); (void)ls;
    for (u32 c = {tid}; c < L; c += {T}) q[c] = {outexpr('p[c]')};
"""
    if gather:
        assert log
        body += f"""
    if ({tid} == 0) {{
        const float* __restrict__ xr = x + (u64)row * L;
        const int t = (int)target[row];
        picked[row] = (u32)t < L ? (xr[t] - m) - ls : 0.0f;           // a target outside the row picks 0
    }}
"""
    extra_params = ", const float* __restrict__ target, float* __restrict__ picked" if gather else ""
    if masked:
        extra_params = ", const float* __restrict__ mask, u32 mrows, float scale"
    src = f"""{PRELUDE}{_row_block_reduce(NW)}
#define E(t) {'(t)' if keep else 'expf((t) - m)'}
extern "C" __global__ __launch_bounds__({threads}) void {name}(const float* __restrict__ x,
        float* __restrict__ out, u32 R, u32 L{extra_params}) {{
    __shared__ float sm[{NW}];
    const u32 row = {row};
    {'' if per_block else 'if (row >= R) return;'}
{body}
}}
"""
    return src, name, _fmt("P", "P", "I", "I", *(("P", "P") if gather else ("P", "I", "f") if masked else ()))



@cache
def ce_grad_rows_kernel(items: int, nt: bool, g_by_value: bool, pow2: bool = False) -> tuple[str, str, str]:
    """Gradient of the summed cross-entropy with respect to 2-D logits whose rows are multiples of
    four floats: out = ((exp((x - max) - logsum) - onehot(target)) * g) / n -- the four kernels of
    CrossEntropy.backward (ops.py:359-370) on a log-softmax rebuilt from the row statistics -- with a
    block per (row, run of 1024 * items columns): the row's three values are read once per block,
    no index is divided, and a thread has `items` 16-byte loads in flight before its first store.
    The same fp32 operations in the same order as the element-wise form of the expression.
    nt: streaming loads and stores (tensors beyond the caches).
    pow2: n is a power of two and the caller passes 1 / n, itself a power of two, in its place: the
    product with it is the quotient, bit for bit (both are the exact value, rounded once), and the
    dozen instructions of an IEEE division per element, a third of the kernel's arithmetic, go."""
    assert items in (1, 2, 4)
    name = f"ce_grad_rows_u{items}" + ("nt" if nt else "") + ("_v" if g_by_value else "_p") + ("_r" if pow2 else "")
    by_n = "* n" if pow2 else "/ n"
    ld = "ld4_stream(reinterpret_cast<const float4*>(xr + c))" if nt else "*reinterpret_cast<const float4*>(xr + c)"
    st = ("{ const v4f ov = {o.x, o.y, o.z, o.w}; __builtin_nontemporal_store(ov, reinterpret_cast<v4f*>(orow + c)); }" if nt
          else "*reinterpret_cast<float4*>(orow + c) = o;")
    garg = "float g" if g_by_value else "const float* __restrict__ gp"
    gval = "" if g_by_value else "    const float g = *gp;\n"
    src = f"""{PRELUDE}
#define ITEMS {items}u
extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ x, const float* __restrict__ row_max,
        const float* __restrict__ row_logsum, const float* __restrict__ target, {garg}, float* __restrict__ out,
        u32 C, u32 runs, float n) {{
    const u32 row = blockIdx.x / runs, c0 = (blockIdx.x - row * runs) * (1024u * ITEMS) + 4u * threadIdx.x;
    const float* __restrict__ xr = x + (u64)row * C;
    float* __restrict__ orow = out + (u64)row * C;
    float4 v[ITEMS];
    #pragma unroll
    for (u32 k = 0; k < ITEMS; ++k) {{ const u32 c = c0 + 1024u * k; if (c < C) v[k] = {ld}; }}
    const float m = row_max[row], ls = row_logsum[row];
    const u32 t = (u32)(int)target[row];
{gval}    #pragma unroll
    for (u32 k = 0; k < ITEMS; ++k) {{
        const u32 c = c0 + 1024u * k;
        if (c < C) {{
            float4 o;
            o.x = ((expf((v[k].x - m) - ls) - (c == t ? 1.0f : 0.0f)) * g) {by_n};
            o.y = ((expf((v[k].y - m) - ls) - (c + 1u == t ? 1.0f : 0.0f)) * g) {by_n};
            o.z = ((expf((v[k].z - m) - ls) - (c + 2u == t ? 1.0f : 0.0f)) * g) {by_n};
            o.w = ((expf((v[k].w - m) - ls) - (c + 3u == t ? 1.0f : 0.0f)) * g) {by_n};
            {st}
        }}
    }}
}}
"""
    return src, name, _fmt("P", "P", "P", "P", "f" if g_by_value else "P", "P", "I", "I", "f")


@cache
def ce_stats_kernel(vec: int, per_block: bool, nt: bool = False, negate: bool = False) -> tuple[str, str, str]:
    """The forward pass of the cross-entropy loss without its log-softmax tensor (ops.py:337-357
    composes max, sub, exp, sum, log, sub over the whole (N, V) logits and gathers one entry per
    row).  Per row r of an (R, L) view: m[r] = max, ls[r] = log(sum(exp(x - m))) and
    picked[r] = (x[r, t] - m) - ls with t = (int)target[r], i.e. the entry the gather of
    cpu_kernel.py:430-441 reads from the log-softmax (0 for a target outside the row).

    One pass over the row, nothing of its size written: 4 B per element + 12 B per row.  Each
    thread walks its items sixteen values at a time with a running maximum and a running sum
    that is rescaled whenever the maximum rises (s <- s * exp(m_old - m_new)), so a row needs
    no second read and no registers of its own: many wavefronts are resident and the exp of one
    overlaps the loads of the others.  The threads' (m, s) pairs are joined the same way.  The
    sum is therefore added in another order than max-then-sum would add it (a few ulp); the
    maximum is exact.  The backward pass rebuilds exp((x - m) - ls) from the logits and these
    two numbers.  One wavefront per row, or one 256-thread block per long row.
    negate: picked[r] is written with its sign flipped, i.e. as the row's loss term, so that the
    loss is a plain sum of it (-(a + b) and (-a) + (-b) are the same float)."""
    nt = nt and vec == 4
    name = f"ce_stats_v{vec}_{'blk' if per_block else 'wav'}{'nt' if nt else ''}{'_neg' if negate else ''}"
    T = "256u" if per_block else "64u"
    tid = "threadIdx.x" if per_block else "(threadIdx.x & 63u)"
    row = "blockIdx.x" if per_block else "(blockIdx.x * 4u + (threadIdx.x >> 6))"
    red_max = "block_max(m, sm)" if per_block else "wave_max(m)"
    red_sum = "block_sum(s, sm)" if per_block else "wave_sum(s)"
    if vec == 4:
        ld = "ld4_stream(p + c)" if nt else "p[c]"
        body = f"""
    const float4* __restrict__ p = reinterpret_cast<const float4*>(x + (u64)row * L);
    const u32 nv = L >> 2;
    float m = NEG_FLT_MAX, s = 0.0f;
    u32 c = {tid};
    for (; c + 3u * {T} < nv; c += 4u * {T}) {{                    // four loads in flight, sixteen values per round
        float4 v[4];
        #pragma unroll
        for (u32 k = 0; k < 4u; ++k) {{ const u32 cc = c + k * {T}; v[k] = {ld.replace('p + c', 'p + cc').replace('p[c]', 'p[cc]')}; }}
        float gm = fmaxf(fmaxf(v[0].x, v[0].y), fmaxf(v[0].z, v[0].w));
        #pragma unroll
        for (u32 k = 1; k < 4u; ++k) gm = fmaxf(gm, fmaxf(fmaxf(v[k].x, v[k].y), fmaxf(v[k].z, v[k].w)));
        if (gm > m) {{ s *= expf(m - gm); m = gm; }}
        #pragma unroll
        for (u32 k = 0; k < 4u; ++k) s += (expf(v[k].x - m) + expf(v[k].y - m)) + (expf(v[k].z - m) + expf(v[k].w - m));
    }}
    for (; c < nv; c += {T}) {{
        const float4 v = {ld};
        const float gm = fmaxf(fmaxf(v.x, v.y), fmaxf(v.z, v.w));
        if (gm > m) {{ s *= expf(m - gm); m = gm; }}
        s += (expf(v.x - m) + expf(v.y - m)) + (expf(v.z - m) + expf(v.w - m));
    }}
"""
    else:
        body = f"""
    const float* __restrict__ p = x + (u64)row * L;
    float m = NEG_FLT_MAX, s = 0.0f;
    for (u32 c = {tid}; c < L; c += {T}) {{
        const float v = p[c];
        if (v > m) {{ s *= expf(m - v); m = v; }}
        s += expf(v - m);
    }}
"""
    src = f"""{PRELUDE}{_row_block_reduce(4)}
extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ x,
        const float* __restrict__ target, float* __restrict__ row_max, float* __restrict__ row_logsum,
        float* __restrict__ picked, u32 R, u32 L) {{
    __shared__ float sm[4];
    const u32 row = {row};
    {'' if per_block else 'if (row >= R) return;'}
{body}
    const float mine = m;
    m = {red_max};
    s *= expf(mine - m);                                          // this thread's sum on the row's scale
    s = {red_sum};
    if ({tid} == 0) {{
        const float ls = logf(s);
        const int t = (int)target[row];
        row_max[row] = m;
        row_logsum[row] = ls;
        const float lp = (u32)t < L ? (x[(u64)row * L + (u32)t] - m) - ls : 0.0f;
        picked[row] = {'-lp' if negate else 'lp'};
    }}
}}
"""
    return src, name, _fmt("P", "P", "P", "P", "P", "I", "I")


def softmax_plan(L: int, vec: int) -> tuple[bool, int, int]:
    """(per_block, nval, threads) for a row of L floats: the register-resident variant with
    the fewest items per thread that holds the row -- one wavefront per row up to 16 items
    per lane, then blocks of 256 and 1024 threads (many waves per CU hide the exp phase
    behind the loads of other rows); (True, 0, 256) streams rows that fit nowhere."""
    items = (L + vec - 1) // vec
    for nval in (1, 2, 4, 8, 16):
        if items <= 64 * nval:
            return False, nval, 256
    for threads, nvals in ((256, (8, 16)), (1024, (8, 16, 32, 64))):
        for nval in nvals:
            if items <= threads * nval:
                return True, nval, threads
    return True, 0, 256


@cache
def softmax_bwd_rows_kernel(vec: int, nval: int, nt: bool = False, masked: bool = False) -> tuple[str, str, str]:
    """dx = y * (g - sum(g * y)) along the contiguous last axis: the backward of a row softmax
    with output y and upstream gradient g, one wavefront per row, both rows held in registers
    (12 B per element instead of the ~36 of the four element-wise and one reduction kernels the
    expression otherwise takes).  Rows of up to 64 * nval items (float4 or float).
    masked: the backward of the scaled, masked form: dx = (mask > 0 ? 0 : y * (g - s)) * scale,
    which is what the backward nodes of softmax, masked_fill and the scalar multiply produce.
    With 16-byte items the mask is read first and items masked in all four lanes (y = 0 there,
    so they add nothing to the sum) are not loaded: a causal mask halves the reads."""
    T, comps, nvx = _rms_lanes(vec)
    nt = nt and vec == 4
    causal = masked == "causal"                           # as in softmax_rows_kernel: the mask is computed from the indices
    masked = bool(masked)
    assert not causal or vec == 4
    name = f"softmax_bwd_rows_v{vec}_r{nval}{'_c' if causal else '_m' if masked else ''}{'nt' if nt else ''}"
    ld = (lambda p: f"ld4_stream({p} + c)") if nt else (lambda p: f"{p}[c]")
    # the row's dot product, with its roundings spelled out (one product, then fused multiply-adds in
    # lane order) so that every variant of this kernel adds the same numbers in the same way
    dot = f"g[k]{comps[0]} * y[k]{comps[0]}"
    for c in comps[1:]:
        dot = f"fmaf(g[k]{c}, y[k]{c}, {dot})"
    skip = masked and vec == 4
    if skip:
        outs = "".join(f"            o{c} = ((mb[k] & {1 << j}u) ? 0.0f : y[k]{c} * (g[k]{c} - s)) * scale;\n"
                       for j, c in enumerate(comps))
        bits = ("mb[k] = (4u * c > last ? 1u : 0u) | (4u * c + 1u > last ? 2u : 0u) | (4u * c + 2u > last ? 4u : 0u) | (4u * c + 3u > last ? 8u : 0u);"
                if causal else
                "const float4 mk = pm[c]; mb[k] = (mk.x > 0.0f ? 1u : 0u) | (mk.y > 0.0f ? 2u : 0u) | (mk.z > 0.0f ? 4u : 0u) | (mk.w > 0.0f ? 8u : 0u);")
        loads = f"""    u32 mb[{nval}];
    #pragma unroll
    for (u32 k = 0; k < {nval}u; ++k) {{
        const u32 c = lane + k * 64u;
        mb[k] = 15u;
        if (c < nv) {{ {bits} }}
    }}
    #pragma unroll
    for (u32 k = 0; k < {nval}u; ++k) {{
        const u32 c = lane + k * 64u;
        y[k] = g[k] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (mb[k] != 15u) {{ y[k] = {ld('py')}; g[k] = {ld('pg')}; }}
    }}
    #pragma unroll
    for (u32 k = 0; k < {nval}u; ++k) if (mb[k] != 15u) s += {dot};
"""
    else:
        if masked:
            # 4-byte form: a masked entry's upstream value is never used (its memory may hold anything)
            outs = f"            const {T} mk = pm[c];\n" + "".join(
                f"            o{c} = (mk{c} > 0.0f ? 0.0f : y[k]{c} * (g[k]{c} - s)) * scale;\n" for c in comps)
            ldg = f"(pm[c] > 0.0f ? 0.0f : {ld('pg')})"
        else:
            outs = "".join(f"            o{c} = y[k]{c} * (g[k]{c} - s);\n" for c in comps)
            ldg = ld('pg')
        loads = f"""    #pragma unroll
    for (u32 k = 0; k < {nval}u; ++k) {{
        const u32 c = lane + k * 64u;
        if (c < nv) {{ y[k] = {ld('py')}; g[k] = {ldg}; s += {dot}; }}
    }}
"""
    st = ("{ const v4f ov = {o.x, o.y, o.z, o.w}; __builtin_nontemporal_store(ov, reinterpret_cast<v4f*>(q) + c); }" if nt
          else "q[c] = o;")
    src = f"""{PRELUDE}
extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ yp,
        const float* __restrict__ gp, float* __restrict__ dx, u32 R, u32 L{", const float* __restrict__ mask, u32 mrows, float scale" if masked else ""}) {{
    const u32 lane = threadIdx.x & 63u;
    const u32 row = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (row >= R) return;
    {"const u32 last = row % mrows;" if causal else f"const {T}* __restrict__ pm = reinterpret_cast<const {T}*>(mask + (u64)(row % mrows) * L);" if masked else ""}
    const {T}* __restrict__ py = reinterpret_cast<const {T}*>(yp + (u64)row * L);
    const {T}* __restrict__ pg = reinterpret_cast<const {T}*>(gp + (u64)row * L);
    {T}* __restrict__ q = reinterpret_cast<{T}*>(dx + (u64)row * L);
    const u32 nv = {nvx};
    {T} y[{nval}], g[{nval}];
    float s = 0.0f;
{loads}    s = wave_sum(s);
    #pragma unroll
    for (u32 k = 0; k < {nval}u; ++k) {{
        const u32 c = lane + k * 64u;
        if (c < nv) {{
            {T} o;
{outs}            {st}
        }}
    }}
}}
"""
    return src, name, _fmt("P", "P", "P", "I", "I", *(("P", "I", "f") if masked else ()))


# =====================================================================================
# random fill
# =====================================================================================

PCG32_MULT = 6364136223846793005


@cache
def uniform_pcg32_kernel() -> tuple[str, str, str]:
    """out[i] = low + (high - low) * f_i (just f_i for low 0, high 1) with f_i = (float)(u_i * 2^-32)
    and u_i the i-th output of PCG32 (XSH-RR 64/32, the generator of cpu_kernel.py:774-874)
    started from `state0` on stream increment `inc`.

    The reference walks the generator sequentially.  Here thread t jumps straight to element
    t (the LCG's state after t steps is state0 * a^t + c * (a^t - 1) / (a - 1), built in
    O(log t) multiplies), emits it, and then strides through the sequence with the
    pre-multiplied step (mstride, pstride) = the LCG advanced by the total thread count.
    Element i therefore holds exactly the value the sequential loop would have written."""
    name = "uniform_pcg32"
    src = f"""{PRELUDE}
static __device__ __forceinline__ u32 pcg_output(u64 s) {{
    const u32 xorshifted = (u32)(((s >> 18u) ^ s) >> 27u);
    const u32 rot = (u32)(s >> 59u);
    return (xorshifted >> rot) | (xorshifted << ((0u - rot) & 31u));
}}
extern "C" __global__ __launch_bounds__(256) void {name}(float* __restrict__ out, u32 n, u64 state0, u64 inc,
        u64 mstride, u64 pstride, float low, float high, u32 affine) {{
    const u32 gid = blockIdx.x * 256u + threadIdx.x;
    const u32 stride = gridDim.x * 256u;
    // jump ahead by gid steps
    u64 acc_mult = 1ull, acc_plus = 0ull, cur_mult = {PCG32_MULT}ull, cur_plus = inc;
    for (u32 d = gid; d != 0u; d >>= 1) {{
        if (d & 1u) {{ acc_mult *= cur_mult; acc_plus = acc_plus * cur_mult + cur_plus; }}
        cur_plus = (cur_mult + 1ull) * cur_plus;
        cur_mult *= cur_mult;
    }}
    u64 s = acc_mult * state0 + acc_plus;
    const float span = high - low;
    for (u64 i = gid; i < n; i += stride) {{
        const float f = (float)pcg_output(s) * 2.3283064365386963e-10f;      // exact: a power of two
        out[i] = affine ? low + span * f : f;
        s = s * mstride + pstride;
    }}
}}
"""
    return src, name, _fmt("P", "I", "Q", "Q", "Q", "Q", "f", "f", "I")


@cache
def u8_to_f32_kernel() -> tuple[str, str, str]:
    """out[i] = (float)bytes[i]: the cast loop of the MNIST idx loaders (cpu_kernel.py:876-1010),
    run after the raw bytes have crossed PCIe (a quarter of the fp32 volume).  Four bytes per
    thread as one 32-bit load and one 16-byte store; `bytes` is 4-byte aligned."""
    name = "u8_to_f32"
    src = f"""{PRELUDE}
extern "C" __global__ __launch_bounds__(256) void {name}(const unsigned char* __restrict__ bytes,
        float* __restrict__ out, u32 n) {{
    const u32 v = blockIdx.x * 256u + threadIdx.x;
    const u32 i = v * 4u;
    if (i + 3u < n) {{
        const u32 w = reinterpret_cast<const u32*>(bytes)[v];
        reinterpret_cast<float4*>(out)[v] = make_float4((float)(w & 255u), (float)((w >> 8) & 255u),
                                                        (float)((w >> 16) & 255u), (float)(w >> 24));
    }} else {{
        for (u32 j = i; j < n; ++j) out[j] = (float)bytes[j];
    }}
}}
"""
    return src, name, _fmt("P", "P", "I")


@cache
def row_store_kernel(pairs: int = 1) -> tuple[str, str, str]:
    """dst[(int)idx[0], :] = src[:] for a (R, W) dst: a row written at a position that is itself
    device data, which is what lets one captured decoding step append to the key/value cache
    at a different place on every replay.  A row index outside [0, R) writes nothing.
    pairs=2: a second (dst, src) of the same shape in the same launch (blockIdx.y picks the pair):
    the key and the value row of one layer."""
    assert pairs in (1, 2)
    name = "row_store" + ("2" if pairs == 2 else "")
    second = ", float* __restrict__ dst2, const float* __restrict__ src2" if pairs == 2 else ""
    pick = "    if (blockIdx.y == 1u) { dst = dst2; src = src2; }\n" if pairs == 2 else ""
    src = f"""{PRELUDE}
extern "C" __global__ __launch_bounds__(256) void {name}(float* __restrict__ dst, const float* __restrict__ src,
        const float* __restrict__ idx, u32 R, u32 W{second}) {{
{pick}    const float fi = idx[0];
    if (!(fi >= 0.0f) || fi >= (float)R) return;
    const u32 row = (u32)fi;
    const u32 j = blockIdx.x * 256u + threadIdx.x;
    if (j < W) dst[(u64)row * W + j] = src[j];
}}
"""
    return src, name, _fmt("P", "P", "P", "I", "I", *(["P", "P"] if pairs == 2 else []))


# =====================================================================================
# fused RMSNorm
# =====================================================================================

def rmsnorm_plan(L: int, vec: int) -> int:
    """Items (float4 or float) each lane of a wavefront keeps for a row of L floats; 0 when
    a row does not fit 16 items per lane (the caller then composes the op from its parts)."""
    items = (L + vec - 1) // vec
    for nval in (1, 2, 3, 4, 6, 8, 12, 16):
        if items <= 64 * nval:
            return nval
    return 0


def _rms_lanes(vec: int) -> tuple[str, tuple, str]:
    """(item type, component suffixes, items-per-row expression) for float4 / float rows."""
    return ("float4", (".x", ".y", ".z", ".w"), "(L >> 2)") if vec == 4 else ("float", ("",), "L")


@cache
def rmsnorm_fwd_kernel(vec: int, nval: int, affine: bool) -> tuple[str, str, str]:
    """y = (x * r) * w with r = 1 / sqrt(sum(x^2) / L + eps) per row of the contiguous last
    axis, and r kept per row for the backward pass: the seven kernels of RMSNorm's
    composition (pow, mean, add, rsqrt, mul, mul; nn/__init__.py:25-41) in one pass that
    reads x once.  One wavefront per row, the row held in registers; same operation order
    per element as the composition, so it differs from it only in the order of the sum."""
    T, comps, nv = _rms_lanes(vec)
    name = f"rmsnorm_fwd_v{vec}_r{nval}{'_w' if affine else ''}"
    sq = " + ".join(f"v[k]{c} * v[k]{c}" for c in comps)
    outs = "".join(f"            o{c} = (v[k]{c} * r){f' * g{c}' if affine else ''};\n" for c in comps)
    src = f"""{PRELUDE}
extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ x,
        const float* __restrict__ w, float* __restrict__ y, float* __restrict__ rinv, u32 R, u32 L, float eps) {{
    const u32 lane = threadIdx.x & 63u;
    const u32 row = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (row >= R) return;
    const {T}* __restrict__ p = reinterpret_cast<const {T}*>(x + (u64)row * L);
    {T}* __restrict__ q = reinterpret_cast<{T}*>(y + (u64)row * L);
    const {T}* __restrict__ wv = reinterpret_cast<const {T}*>(w); (void)wv;
    const u32 nv = {nv};
    {T} v[{nval}];
    float ss = 0.0f;
    #pragma unroll
    for (u32 k = 0; k < {nval}u; ++k) {{
        const u32 c = lane + k * 64u;
        if (c < nv) {{ v[k] = p[c]; ss += {sq}; }}
    }}
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / (float)L + eps);
    if (lane == 0) rinv[row] = r;
    #pragma unroll
    for (u32 k = 0; k < {nval}u; ++k) {{
        const u32 c = lane + k * 64u;
        if (c < nv) {{
            {f'const {T} g = wv[c];' if affine else ''}
            {T} o;
{outs}            q[c] = o;
        }}
    }}
}}
"""
    return src, name, _fmt("P", "P", "P", "P", "I", "I", "f")


@cache
def rmsnorm_bwd_kernel(vec: int, nval: int, affine: bool, through_mean: bool, plus: bool = False) -> tuple[str, str, str]:
    """Backward of the fused RMSNorm.  Per row, with dn = dy * w:
        dx = dn * r                                         (the path through x * r)
           + (x * 2) * ((1/L) * (sum(dn * x) * (r^3 * -0.5)))   (the path through mean(x^2)),
    the second term only when through_mean: the reference's Mean.backward scales by
    full(1/N), whose fill value is truncated to int 0 (ops.py:86-91, cpu.py:252), so its
    RMSNorm passes no gradient through the normaliser.
    dw = sum over rows of dy * (x * r): each wavefront walks rows_per_wave consecutive rows
    with its columns' partial sums in registers and writes one row of `dwpart`; a column
    reduction over those partial rows finishes it.
    plus: what is stored is prev + dx for a given array prev shaped like x (a gradient that
    reached x by another route, e.g. the residual connection around the norm): dx is rounded to
    fp32 first, so the sum has the bits of a separate addition kernel."""
    T, comps, nv = _rms_lanes(vec)
    name = f"rmsnorm_bwd_v{vec}_r{nval}{'_w' if affine else ''}{'_m' if through_mean else ''}{'_p' if plus else ''}"
    dn = lambda c: f"(d[k]{c} * g[k]{c})" if affine else f"d[k]{c}"          # noqa: E731
    dot = " + ".join(f"{dn(c)} * v[k]{c}" for c in comps)
    dxs = "".join(
        f"                o{c} = {dn(c)} * r" + (f" + (v[k]{c} * 2.0f) * coef" if through_mean else "") + ";\n"
        for c in comps)
    accs = "".join(f"                acc[k]{c} += d[k]{c} * (v[k]{c} * r);\n" for c in comps) if affine else ""
    zero = "float4{0.0f, 0.0f, 0.0f, 0.0f}" if vec == 4 else "0.0f"
    tail = f"""    {T}* __restrict__ pw = reinterpret_cast<{T}*>(dwpart + (u64)wid * L);
    #pragma unroll
    for (u32 k = 0; k < {nval}u; ++k) {{ const u32 c = lane + k * 64u; if (c < nv) pw[c] = acc[k]; }}""" if affine else ""
    plus_load = f"""
        {T} e[{nval}];
        #pragma unroll
        for (u32 k = 0; k < {nval}u; ++k) {{
            const u32 c = lane + k * 64u;
            if (c < nv) e[k] = reinterpret_cast<const {T}*>(prev + (u64)row * L)[c];
        }}""" if plus else ""
    # the empty asm keeps the last multiply of dx from being contracted into this addition
    plus_add = "".join(f'                asm volatile("" : "+v"(o{c}));\n                o{c} = e[k]{c} + o{c};\n' for c in comps) if plus else ""
    src = f"""{PRELUDE}
extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ x,
        const float* __restrict__ w, const float* __restrict__ rinv, const float* __restrict__ dy,
        float* __restrict__ dx, float* __restrict__ dwpart, u32 R, u32 L, u32 rows_per_wave{', const float* __restrict__ prev' if plus else ''}) {{
    const u32 lane = threadIdx.x & 63u;
    const u32 wid = blockIdx.x * 4u + (threadIdx.x >> 6);
    const u32 row0 = wid * rows_per_wave;
    if (row0 >= R) return;
    const u32 nv = {nv};
    {T} g[{nval}], acc[{nval}]; (void)g; (void)acc;
    #pragma unroll
    for (u32 k = 0; k < {nval}u; ++k) {{
        const u32 c = lane + k * 64u;
        acc[k] = {zero};
        {f'if (c < nv) g[k] = reinterpret_cast<const {T}*>(w)[c];' if affine else '(void)c;'}
    }}
    const u32 row1 = min(row0 + rows_per_wave, R);
    for (u32 row = row0; row < row1; ++row) {{
        const {T}* __restrict__ p = reinterpret_cast<const {T}*>(x + (u64)row * L);
        const {T}* __restrict__ pd = reinterpret_cast<const {T}*>(dy + (u64)row * L);
        {T}* __restrict__ q = reinterpret_cast<{T}*>(dx + (u64)row * L);
        const float r = rinv[row];
        {T} v[{nval}], d[{nval}];
        float s = 0.0f; (void)s;
        #pragma unroll
        for (u32 k = 0; k < {nval}u; ++k) {{
            const u32 c = lane + k * 64u;
            if (c < nv) {{ v[k] = p[c]; d[k] = pd[c]; {f's += {dot};' if through_mean else ''} }}
        }}{plus_load}
        {'s = wave_sum(s);' if through_mean else ''}
        const float coef = (1.0f / (float)L) * (s * ((r * r * r) * -0.5f)); (void)coef;
        #pragma unroll
        for (u32 k = 0; k < {nval}u; ++k) {{
            const u32 c = lane + k * 64u;
            if (c < nv) {{
                {T} o;
{dxs}{plus_add}                q[c] = o;
{accs}            }}
        }}
    }}
{tail}
}}
"""
    return src, name, _fmt("P", "P", "P", "P", "P", "P", "I", "I", "I", *(["P"] if plus else []))


# =====================================================================================
# matmul
# =====================================================================================

MATMUL_LDS_LIMIT = 160 * 1024          # LDS per CU on gfx950, all of it available to one block


def matmul_lds_bytes(WM: int, WN: int, MI: int, NJ: int, BK: int, ta: bool = False, tb: bool = False, S: int = 32) -> int:
    """Static LDS of one block (both operands, double-buffered)."""
    BM, BN = S * MI * WM, S * NJ * WN
    a = BK * BM if ta else BM * (BK + 4)
    b = BN * (BK + 4) if tb else BK * BN
    return 2 * 4 * (a + b)


MATMUL_TRI = ("", "out_lower", "a_lower", "at_lower")


@cache
def matmul_groups_fit(WM: int, WN: int, MI: int, NJ: int, BK: int, ta: bool, tb: bool, S: int, G: int) -> bool:
    """Whether a block of G k-groups of this tile exists: at most 1024 threads, and LDS for G sets of operand buffers plus
    the groups' partial tiles where those do not fit into A's buffers."""
    BM, BN = S * MI * WM, S * NJ * WN
    red_in_a = (G - 1) * BM * BN <= 2 * G * (BK * BM if ta else BM * (BK + 4))
    return (G * 64 * WM * WN <= 1024 and
            G * matmul_lds_bytes(WM, WN, MI, NJ, BK, ta, tb, S) + (0 if red_in_a else (G - 1) * 4 * BM * BN) <= MATMUL_LDS_LIMIT)


def matmul_kernel(WM: int, WN: int, MI: int, NJ: int, BK: int, veca: bool, vecb: bool,
                  ta: bool = False, tb: bool = False, tri: str = "", strided: bool = False,
                  epi: str = "", S: int = 32, norm: bool = False, splitk: bool = False, exact: bool = False,
                  kgroups: int = 1, deep: bool = False) -> tuple[str, str, str]:
    """C[z] = op(A[z]) . op(B[z]), fp32, row-major, on the matrix cores (v_mfma_f32_32x32x2_f32, or
    v_mfma_f32_16x16x4_f32 for S = 16).

    Replaces the i-k-j loops of cpu_kernel.py:351-428.  Batched over blockIdx.z with two
    batch extents (z = zb * nbc + zc) whose operand strides may be 0, which is how the
    reference broadcasts a batch or channel dim (cpu.py:519-532, :553-559).
    ta: A is given transposed, as a (K, M) row-major array; tb: B is given transposed, as
    (N, K).  These read in place what MatMul.backward and Linear otherwise materialise with a
    permute kernel (ops.py:308-335, tensor.py:549-563); the k terms of every output element
    are added in the same order in all variants, so the results are bit-identical.

    Tiling.  A block of WM x WN wavefronts owns a (32*MI*WM) x (32*NJ*WN) tile of C; each
    wavefront owns MI x NJ MFMA tiles of 32x32, i.e. 16*MI*NJ accumulator registers.  The
    K loop advances BK at a time through double-buffered LDS (one barrier per step; the
    next A/B tiles are in flight in registers while the current ones are multiplied).

    An operand whose global rows run along k (A, or B when tb) sits in LDS as [row][k] with a
    4-float pad; one 32x32x2 MFMA consumes, per lane, X[row = lane%32][k = lane/32], and the
    k order inside a group of 8 is permuted (lane half h takes k = 8*blk + 4*h + s at step s,
    for both operands alike), so one ds_read_b128 per lane feeds four MFMA steps.
    An operand whose global rows run along the output dim (B, or A when ta) sits in LDS as
    [k][col]; the tiles a wavefront owns along that dim interleave (lane c of tile j owns
    col NJ*c + j), so one read of NJ consecutive floats feeds NJ MFMAs, and for B the
    epilogue then holds NJ adjacent columns of a row per lane: one dwordx4 store for NJ = 4,
    a coalesced 512-byte row segment per half wave.
    veca / vecb: 16-byte global loads of A / of B (the contiguous extent is a multiple of 4
    and bases and batch strides are 16-byte aligned); vecb and not tb also means 16-byte
    stores of C.  Out-of-range rows, columns and k are read as zero and never written.
    Blocks are renumbered so that the eight XCDs (round-robin dispatch) each work on a
    contiguous band of C tiles, walked in groups of 8 tile rows for L2 reuse.
    tri: square (T x T) structure the caller vouches for, per batch entry; the skipped work is
    products with exact zeros or output nobody reads, so the kept results keep their bits:
      out_lower  only output tiles that touch n <= m are computed (the others are left unwritten)
      a_lower    op(A) = A is lower triangular (A[m][k] = 0 for k > m): k stops at the tile's last row
      at_lower   op(A) = A^T with the stored A (K x M) lower triangular: k starts at the tile's first row
    epi: what the epilogue does to each result c on its way to memory, with e the entry at the same place of a
    fourth operand E shaped like C: "add" stores c + e (a residual), "relu" stores max-like c > 0 ? c : 0,
    "gate" stores e > 0 ? c : 0 (the backward of a ReLU whose output is E).  One rounding each, as the
    separate element-wise kernel would do.  "bias": E is one row of N values, added to every row of C (the
    bias of a linear layer, tensor.py:549-563: the Add node after the product, as the product is stored).
    S: edge of the MFMA tile.  A wavefront's share of one output element's k sum is a fixed chain of
    MFMA steps however small its tile, so a long-k product with few output tiles (2048 x 128 x 512: 64
    tiles of 64x64) is bound by that chain on a quarter of the SIMDs.  S = 16 gives every wavefront a
    (16*MI) x (16*NJ) tile, four times as many wavefronts and a quarter of the chain each.  One 16x16x4
    step adds four k; the lane groups take k = 8*blk + {0, 4, 1, 5} and then {2, 6, 3, 7}, the order
    in which two 32x32x2 steps at a time add them.
    strided: A, B and C have their own row pitches (lda, ldb, ldc, in floats) and C its own two batch
    strides, so operands and result can be matrices cut out of larger tensors -- the heads of a
    (B, T, h*d) projection are (T x d) matrices with pitch h*d, batch strides T*h*d and d.
    norm: the rows of A are RMS-normalised on their way into the product -- (a * r) * gain with
    r = 1 / sqrt(sum(a^2) / K + eps) per row -- for K <= BK, where a block's A tile holds whole rows:
    once the tile is in LDS, each wavefront takes rows of it, a lane one 16-byte item, and rewrites them
    with the statements of rmsnorm_fwd_kernel, so the product sees the values that kernel would have
    stored.  The blocks of the first tile column also write the normalised rows to yn and r to rinv
    (what the backward pass of the norm and of the product need) unless yn is null.  Arguments after
    the others: gain, eps, yn, rinv.
    splitk: the k sum is cut into gridDim.y slices of kchunk (a multiple of BK) and block (x, y, z) adds slice y
    of tile x: a product with few output tiles and a long k (the weight gradient of a linear layer is a handful
    of tiles with k = the number of tokens) then fills the chip.  Each block writes its partial tile to slab
    (z * gridDim.y + y) of a workspace W of gridDim.z * gridDim.y * M * N floats instead of C, and a column-sum
    launch over the slabs finishes the product.  An output element is then a sum of per-slice sums: not the
    bits of the unsplit kernel (each slice still adds its k in that kernel's order), within the 1e-4 that
    products are held to.  (Folding the slabs in the same launch, by the block that finishes a tile last, was
    measured and dropped: the device-wide fence in front of the arrival counter cost 50 us per launch.)
    Arguments after the others: W, kchunk.
    exact: the launcher vouches that M, N and K are whole multiples of the tile (and kchunk of BK, and K of kchunk).  The k
    loop then has no conditional part: no load carries a bounds test or a zero select (loader threads that fall outside
    the tile in a pass skip the load as they skip the store; inside the tile every address is inside the matrix), and
    the last step fetches its own tiles once more instead of branching around the fetch.  A scheduling fence keeps the
    fetch in front of the MFMA run (left alone, the compiler sinks the loads to their use and waits for them there).
    Same loads, same products: same bits; 4096^3 118.6 -> 133.4 TFLOP/s, 2048^3 101.0 -> 108.5, 1024^3 75.8 -> 82.6,
    8192^3 135.3 -> 137.3 in one run.
    kgroups: G > 1 cuts the k sum into G slices *inside a block*: the block has G times the wavefronts, group q of them runs
    the whole k loop of the tile over k in [q * kchunk, (q + 1) * kchunk) with LDS buffers of its own, and at the end the
    groups' partial tiles meet in LDS and group 0 adds them in group order and stores.  For an output of few tiles this puts
    G wavefronts on every SIMD of the CUs that have a block, so one group's LDS and memory latency is covered by another's
    MFMA run -- what a second launch over slabs cannot give a product that already has a block on every CU.  All groups take
    the same number of k steps (they share the barriers); steps beyond K read zeros.  The sum is added in a fixed order of its
    own (slice by slice), like the split-k form.  Arguments after the others: kchunk (a multiple of BK).
    deep: the k loop as a software pipeline two steps deep.  The tiles of step t + 2 are fetched during step t into a second
    set of registers, and the LDS stores of the tiles of step t + 1 are issued between the MFMA steps of the second half of
    step t instead of behind them (the fetches, with their address arithmetic and bounds tests, between those of the first
    half; the LDS reads of each group of 8 k one group ahead of its MFMA steps).  A wavefront issues in order: whatever
    follows a run of dependent MFMA steps waits for the run, but an instruction placed between two of them is issued while
    the first one executes.  Scheduling fences pin the order.  Measured beforehand by taking parts of the step away: at
    4096^3 the fetches' latency cost 7 % of the launch and the LDS stores 5 %, at 1024^3 11 % each; with this form 1024^3
    24.2 -> 20.6 us, 2048^3 152.8 -> 136.4, 4096^3 1047 -> 998, 512^3 7.7 -> 6.7, (768 x 1024)^T (1024 x 3072) 56.7 -> 49.5.
    The step past the last one fetches the last tiles again instead of branching.  Same loads, same MFMA steps in the same
    order: same bits.
    """
    BM, BN, T = S * MI * WM, S * NJ * WN, 64 * WM * WN
    G = kgroups
    assert isinstance(splitk, bool) and not (splitk and (tri or strided or epi or norm))
    assert G in (1, 2, 3, 4, 8, 16) and not (G > 1 and (splitk or tri or strided or epi or norm))
    NE = S * S // 64                                        # accumulator registers per MFMA tile
    assert BK % 8 == 0 and MI in (1, 2, 3, 4) and NJ in (1, 2, 3, 4) and S in (16, 32) and G * T <= 1024
    red_in_a = (G - 1) * BM * BN <= 2 * G * (BK * BM if ta else BM * (BK + 4))       # the partial tiles of the groups reuse A's LDS buffers if they fit
    assert matmul_groups_fit(WM, WN, MI, NJ, BK, ta, tb, S, G)
    name = (f"matmul_{BM}x{BN}x{BK}_w{WM}x{WN}_{'a4' if veca else 'a1'}{'b4' if vecb else 'b1'}"
            f"{'_tn' if ta else ''}{'_nt' if tb else ''}{'_' + tri if tri else ''}{'_ld' if strided else ''}{'_' + epi if epi else ''}{'_m16' if S == 16 else ''}")
    assert tri in MATMUL_TRI and not (tri == "a_lower" and ta) and not (tri == "at_lower" and not ta)
    assert not norm or (veca and not ta and not tri and not strided and BK <= 256)
    if norm:
        name += "_rms"
    if splitk:
        name += "_sk"
    if G > 1:
        name += f"_g{G}"
    if deep:
        assert not norm
        name += "_d"
    if exact:
        assert veca and vecb and not norm
        name += "_x"
    comp = ["x", "y", "z", "w"]
    vtype = {1: "float", 2: "float2", 3: "f3v", 4: "float4"}

    def loader(X: str, along_k: bool, rows_name: str, R: int, ld: str, ext: str, base: str, vec: bool):
        """Global -> registers -> LDS for operand X (A or B).
        along_k: global rows run along k: element (row, k) at X[row * K + k]; LDS [row][k].
        else:    global rows run along the output dim: element (k, col) at X[k * ld + col]; LDS [k][col].
        Loader threads walk the tile in passes; a tile extent that is no multiple of the pass
        is cut off by a guard, and threads beyond the last whole row repeat a neighbour's
        element (same address, same value)."""
        x = X.lower()
        if along_k:
            Q = BK // 4
            assert T % Q == 0
            rpp = T // Q                                   # tile rows per pass
            P = -(-R // rpp)
            guard = f"if ({x}_r + p * {rpp}u < {R}u) " if R % rpp else ""
            idx = f"const u32 {x}_q = tid % {Q}u, {x}_r = tid / {Q}u;"
            where = f"const u32 row = {base} + {x}_r + p * {rpp}u, k = k0 + 4u * {x}_q;"
            if vec:
                ld_code = (f"{guard}{{ const v4f t_ = *reinterpret_cast<const v4f*>({X} + (u64)row * g.K + k); r{x}[p] = make_float4(t_.x, t_.y, t_.z, t_.w); }}" if exact else
                           f"r{x}[p] = (row < g.{ext} && k < KEND) ? *reinterpret_cast<const float4*>({X} + (u64)row * g.K + k)\n"
                           f"                                         : make_float4(0.f, 0.f, 0.f, 0.f);")
            else:
                ld_code = (f"const float* __restrict__ s = {X} + (u64)row * g.K + k;\n"
                           f"            const bool ok = row < g.{ext};\n" +
                           "".join(f"            r{x}[p].{c} = (ok && k + {n}u < KEND) ? s[{n}] : 0.f;\n" for n, c in enumerate(comp)))
            st = f"{guard}*reinterpret_cast<float4*>(&{X}s[buf][{x}_r + p * {rpp}u][4u * {x}_q]) = r{x}[p];"
            decl = f"__shared__ __attribute__((aligned(16))) float {X}s[{2 * G}][{R}][{BK + 4}];"
        else:
            Q = R // 4
            assert T >= Q
            rpp = T // Q                                   # k rows per pass
            P = -(-BK // rpp)
            guard = f"if ({x}_r + p * {rpp}u < BK) " if (BK % rpp or T % Q) else ""
            idx = f"const u32 {x}_q = tid % {Q}u, {x}_r = tid / {Q}u;"
            where = f"const u32 k = k0 + {x}_r + p * {rpp}u, col = {base} + 4u * {x}_q;"
            if vec:
                ld_code = (f"{guard}{{ const v4f t_ = *reinterpret_cast<const v4f*>({X} + (u64)k * g.{ext} + col); r{x}[p] = make_float4(t_.x, t_.y, t_.z, t_.w); }}" if exact else
                           f"r{x}[p] = (k < KEND && col < g.{ext}) ? *reinterpret_cast<const float4*>({X} + (u64)k * g.{ext} + col)\n"
                           f"                                         : make_float4(0.f, 0.f, 0.f, 0.f);")
            else:
                ld_code = (f"const float* __restrict__ s = {X} + (u64)k * g.{ext} + col;\n"
                           f"            const bool ok = k < KEND;\n" +
                           "".join(f"            r{x}[p].{c} = (ok && col + {n}u < g.{ext}) ? s[{n}] : 0.f;\n" for n, c in enumerate(comp)))
            st = f"{guard}*reinterpret_cast<float4*>(&{X}s[buf][{x}_r + p * {rpp}u][4u * {x}_q]) = r{x}[p];"
            decl = f"__shared__ __attribute__((aligned(16))) float {X}s[{2 * G}][{BK}][{R}];"
        load = f"""        #pragma unroll
        for (u32 p = 0; p < {P}u; ++p) {{
            {where}
            {ld_code}
        }}
"""
        stash = f"""        #pragma unroll
        for (u32 p = 0; p < {P}u; ++p)
            {st}
"""
        def ld_piece(rs: int, pi: int, k0: str) -> str:           # pass pi of the fetch into register set rs
            return f"            {{ const u32 p = {pi}u, k0 = {k0}; {where} {ld_code} }}\n".replace(f"r{x}[p]", f"r{x}{rs}[p]")

        def st_piece(rs: int, pi: int, buf: str) -> str:          # pass pi of register set rs into LDS buffer buf
            return f"            {{ const u32 p = {pi}u, buf = {buf}; {st} }}\n".replace(f"r{x}[p]", f"r{x}{rs}[p]")
        return decl, idx, P, load, stash, ld_piece, st_piece

    decl_a, idx_a, PA, load_a, stash_a, ld_piece_a, st_piece_a = loader("A", not ta, "M", BM, "M", "M", "m0", veca)
    decl_b, idx_b, PB, load_b, stash_b, ld_piece_b, st_piece_b = loader("B", tb, "N", BN, "N", "N", "n0", vecb)

    # ---- the multiply: one group of 8 k per iteration, four 32x32x2 (two 16x16x4) MFMA steps
    pre = ""
    if not ta:
        pre += (f"            float4 a[MI];\n            #pragma unroll\n            for (int i = 0; i < MI; ++i)\n"
                f"                a[i] = *reinterpret_cast<const float4*>(&As[buf][wm0 + {S}u * i + r][kb + 4u * {'h' if S == 32 else '(h & 1u)'}]);\n")
    if tb:
        pre += (f"            float4 b[NJ];\n            #pragma unroll\n            for (int j = 0; j < NJ; ++j)\n"
                f"                b[j] = *reinterpret_cast<const float4*>(&Bs[buf][wn0 + {S}u * j + r][kb + 4u * {'h' if S == 32 else '(h & 1u)'}]);\n")
    mfma = pre
    for st_ in range(4 if S == 32 else 2):
        # the k (within the group of 8) that this lane feeds to step st_, and the component of a float4 read at 4*(k/4)
        krow = f"kb + 4u * h + {st_}u" if S == 32 else f"kb + 4u * (h & 1u) + (h >> 1) + {2 * st_}u"
        pick = (lambda v: f"{v}.{comp[st_]}") if S == 32 else (lambda v: f"((h >> 1) ? {v}.{comp[2 * st_ + 1]} : {v}.{comp[2 * st_]})")
        mfma += "            {\n"
        if ta:
            mfma += (f"              const {vtype[MI]} av = *reinterpret_cast<const {vtype[MI]}*>"
                     f"(&As[buf][{krow}][wm0 + {MI}u * r]);\n")
        if not tb:
            mfma += (f"              const {vtype[NJ]} bv = *reinterpret_cast<const {vtype[NJ]}*>"
                     f"(&Bs[buf][{krow}][wn0 + {NJ}u * r]);\n")
        for i_ in range(MI):
            ai = (("av" if MI == 1 else f"av.{comp[i_]}") if ta else pick(f"a[{i_}]"))
            for j_ in range(NJ):
                bj = (pick(f"b[{j_}]") if tb else ("bv" if NJ == 1 else f"bv.{comp[j_]}"))
                mfma += (f"              acc[{i_}][{j_}] = __builtin_amdgcn_mfma_f32_{'32x32x2' if S == 32 else '16x16x4'}f32("
                         f"{ai}, {bj}, acc[{i_}][{j_}], 0, 0, 0);\n")
        mfma += "            }\n"

    if deep:
        NSTEP = 4 if S == 32 else 2
        hk = "h" if S == 32 else "(h & 1u)"

        def krow_at(kb: str, st_: int) -> str:
            return f"{kb} + 4u * h + {st_}u" if S == 32 else f"{kb} + 4u * (h & 1u) + (h >> 1) + {2 * st_}u"

        def reads(P: str, kb: str) -> str:
            out = ""
            if not ta:
                out += "".join(f"                fa[{P}][{i}] = *reinterpret_cast<const float4*>(&As[buf][wm0 + {S}u * {i} + r][{kb} + 4u * {hk}]);\n" for i in range(MI))
            if tb:
                out += "".join(f"                fb[{P}][{j}] = *reinterpret_cast<const float4*>(&Bs[buf][wn0 + {S}u * {j} + r][{kb} + 4u * {hk}]);\n" for j in range(NJ))
            for st_ in range(NSTEP):
                if ta:
                    out += f"                fav[{P}][{st_}] = *reinterpret_cast<const {vtype[MI]}*>(&As[buf][{krow_at(kb, st_)}][wm0 + {MI}u * r]);\n"
                if not tb:
                    out += f"                fbv[{P}][{st_}] = *reinterpret_cast<const {vtype[NJ]}*>(&Bs[buf][{krow_at(kb, st_)}][wn0 + {NJ}u * r]);\n"
            return out

        steps, step_lines = "", []
        for st_ in range(NSTEP):
            pick = (lambda v: f"{v}.{comp[st_]}") if S == 32 else (lambda v: f"((h >> 1) ? {v}.{comp[2 * st_ + 1]} : {v}.{comp[2 * st_]})")
            for i_ in range(MI):
                ai = ((f"fav[P][{st_}]" if MI == 1 else f"fav[P][{st_}].{comp[i_]}") if ta else pick(f"fa[P][{i_}]"))
                for j_ in range(NJ):
                    bj = (pick(f"fb[P][{j_}]") if tb else (f"fbv[P][{st_}]" if NJ == 1 else f"fbv[P][{st_}].{comp[j_]}"))
                    step_lines.append(f"            acc[{i_}][{j_}] = __builtin_amdgcn_mfma_f32_{'32x32x2' if S == 32 else '16x16x4'}f32("
                                      f"{ai}, {bj}, acc[{i_}][{j_}], 0, 0, 0);\n")
        steps = "".join(step_lines)
        frag_decl = (("" if ta else f"        float4 fa[2][{MI}];\n") + (f"        float4 fb[2][{NJ}];\n" if tb else "") +
                     (f"        {vtype[MI]} fav[2][{NSTEP}];\n" if ta else "") + ("" if tb else f"        {vtype[NJ]} fbv[2][{NSTEP}];\n"))
    mfma_run = f"""        #pragma unroll
        for (u32 kb = 0; kb < BK; kb += 8u) {{
{mfma}        }}"""

    def deep_step(cb: int, ls: int, ss: int, k0: str) -> str:
        """One k step of the deep form: MFMA steps on LDS buffer cb; the fetch of the tiles at k0 into register set ls is spread
        over the first half of the MFMA steps, the LDS stores of register set ss into buffer cb ^ 1 over the second half."""
        FENCE = "            __builtin_amdgcn_sched_barrier(0);\n"
        groups = BK // 8
        half = max(1, groups // 2)
        fetch = [ld_piece_a(ls, p_, k0) for p_ in range(PA)] + [ld_piece_b(ls, p_, k0) for p_ in range(PB)]
        lds = (lambda b_: f"gb + {b_}u") if G > 1 else (lambda b_: f"{b_}u")          # (a k-group has its own pair of buffers)
        store = [st_piece_a(ss, p_, lds(cb ^ 1)) for p_ in range(PA)] + [st_piece_b(ss, p_, lds(cb ^ 1)) for p_ in range(PB)]

        def spread(lines: list, extras: list) -> str:
            # an extra after every n-th MFMA step, the first one behind the first step (which is then executing)
            if not extras:
                return "".join(lines)
            n = max(1, len(lines) // len(extras))
            out, e = "", 0
            for at, line in enumerate(lines):
                out += line
                if at % n == 0 and e < len(extras):
                    out += FENCE + extras[e] + FENCE
                    e += 1
            return out + "".join(FENCE + x for x in extras[e:])
        code = f"        {{   // MFMA steps on buffer {cb}; fetch into register set {ls}; register set {ss} into buffer {cb ^ 1}\n            const u32 buf = {lds(cb)};\n"
        code += reads("0", "0u")
        first = [(g_, l_) for g_ in range(half) for l_ in step_lines]
        second = [(g_, l_) for g_ in range(half, groups) for l_ in step_lines]
        for part, extras in ((first, fetch), (second, store)):
            # the lines of a group carry the operand set of the group; the reads of the next group go in front of the group's first step
            lines = []
            for at, (g_, l_) in enumerate(part):
                head = ""
                if at % len(step_lines) == 0 and g_ + 1 < groups:
                    head = reads(f"{(g_ + 1) & 1}", f"{8 * (g_ + 1)}u") + FENCE
                lines.append(head + l_.replace("[P]", f"[{g_ & 1}]"))
            code += spread(lines, extras)
        return code + "        }\n"


    # ---- epilogue: accumulator e of tile (i, j) belongs to operand-row index 8*(e/4) + 4*h + e%4
    # (4*h + e for the 16-wide tile) of A's tile i and operand-row index lane%S of B's tile j
    arow = "8u * (e >> 2) + 4u * h + (e & 3)" if S == 32 else "4u * h + e"
    row_expr = (f"m0 + wm0 + {MI}u * ({arow}) + i" if ta else f"m0 + wm0 + {S}u * i + {arow}")
    if tb:
        store = f"""                #pragma unroll
                for (int j = 0; j < NJ; ++j) {{ const u32 col = n0 + wn0 + {S}u * j + r; if (col < g.N) crow[col] = acc[i][j][e]; }}"""
    elif vecb and NJ == 4:
        store = f"""                const u32 col = n0 + wn0 + {NJ}u * r;
                if (col + 3u < g.N) {{
                    *reinterpret_cast<float4*>(crow + col) =
                        make_float4(acc[i][0][e], acc[i][1][e], acc[i][2][e], acc[i][3][e]);
                }} else {{
                    #pragma unroll
                    for (int j = 0; j < NJ; ++j) if (col + j < g.N) crow[col + j] = acc[i][j][e];
                }}"""
    else:
        store = f"""                const u32 col = n0 + wn0 + {NJ}u * r;
                #pragma unroll
                for (int j = 0; j < NJ; ++j) if (col + j < g.N) crow[col + j] = acc[i][j][e];"""

    # a triangular job makes the tile rows unequal (short near one end of the diagonal, long at the other)
    # and consecutive blocks go to consecutive XCDs: rotating the row by the batch index keeps one XCD
    # from collecting all the long rows
    m0n0 = ("    const u32 m0 = ((tm + blockIdx.z) % tiles_m) * BM, n0 = tn * BN;" if tri
            else "    const u32 m0 = tm * BM, n0 = tn * BN;")
    skip_tile = "    if (n0 > m0 + BM - 1u) return;                    // the whole tile lies above the diagonal\n" if tri == "out_lower" else ""
    norm_code = ""
    if norm:
        norm_code = f"""    {{   // every k of a row is in this tile (the launcher vouches for K <= BK): normalise the rows where they lie
        const u32 K4 = g.K >> 2;
        const bool keep = tn == 0u && yn != nullptr;          // one tile column writes what the backward pass needs
        #pragma unroll
        for (u32 rr = wave; rr < BM; rr += {WM * WN}u) {{           // (the rows of a wavefront are independent: their chains overlap)
            float4 av = make_float4(0.f, 0.f, 0.f, 0.f);
            float ss = 0.0f;
            if (lane < K4) {{ av = *reinterpret_cast<const float4*>(&As[0][rr][4u * lane]); ss += av.x * av.x + av.y * av.y + av.z * av.z + av.w * av.w; }}
            ss = wave_sum(ss);
            const float rs = 1.0f / sqrtf(ss / (float)g.K + eps);
            if (lane < K4) {{
                const float4 gn = reinterpret_cast<const float4*>(gain)[lane];
                float4 o;
                o.x = (av.x * rs) * gn.x; o.y = (av.y * rs) * gn.y; o.z = (av.z * rs) * gn.z; o.w = (av.w * rs) * gn.w;
                *reinterpret_cast<float4*>(&As[0][rr][4u * lane]) = o;
                if (keep && m0 + rr < g.M) reinterpret_cast<float4*>(yn + (u64)(m0 + rr) * g.K)[lane] = o;
            }}
            if (keep && lane == 0u && m0 + rr < g.M) rinv[m0 + rr] = rs;
        }}
    }}
    __syncthreads();
"""
    if G > 1:
        kloop = f"""    const u32 kt0 = kbeg / BK, nk = kt0 + kchunk / BK;         // every group takes the same number of steps: they share the barriers
    const u32 gb = 2u * grp;                                      // this group's pair of LDS buffers
    load_tiles(kt0 * BK);
    stash_tiles(gb);
    __syncthreads();
    for (u32 kt = kt0; kt < nk; ++kt) {{
        const u32 buf = gb + ((kt - kt0) & 1u);"""
    elif splitk:
        kloop = f"""    const u32 nk = (kend + BK - 1u) / BK, kt0 = kbeg / BK;                 // this block's slice of k
    load_tiles(kt0 * BK);
    stash_tiles(0u);
    __syncthreads();
    for (u32 kt = kt0; kt < nk; ++kt) {{
        const u32 buf = (kt - kt0) & 1u;"""
    elif tri in ("", "out_lower"):
        kloop = f"""    const u32 nk = (g.K + BK - 1u) / BK;
    load_tiles(0u);
    stash_tiles(0u);
    __syncthreads();
{norm_code}    for (u32 kt = 0; kt < nk; ++kt) {{
        const u32 buf = kt & 1u;"""
    else:
        krange = {"a_lower": "const u32 nk = (min(g.K, m0 + BM) + BK - 1u) / BK, kt0 = 0u;       // A is zero right of the diagonal",
                  "at_lower": "const u32 nk = (g.K + BK - 1u) / BK, kt0 = m0 / BK;                 // the stored A is zero above the diagonal"}[tri]
        kloop = f"""    {krange}
    load_tiles(kt0 * BK);
    stash_tiles(0u);
    __syncthreads();
    for (u32 kt = kt0; kt < nk; ++kt) {{
        const u32 buf = (kt - kt0) & 1u;"""
    if deep:
        if G > 1:
            krange = "const u32 kt0 = kbeg / BK, nk = kt0 + kchunk / BK, gb = 2u * grp;      // every group takes the same number of steps: they share the barriers"
        elif splitk:
            krange = "const u32 nk = (kend + BK - 1u) / BK, kt0 = kbeg / BK;                 // this block's slice of k"
        elif tri in ("", "out_lower"):
            krange = "const u32 nk = (g.K + BK - 1u) / BK, kt0 = 0u;"
        else:
            krange = {"a_lower": "const u32 nk = (min(g.K, m0 + BM) + BK - 1u) / BK, kt0 = 0u;       // A is zero right of the diagonal",
                      "at_lower": "const u32 nk = (g.K + BK - 1u) / BK, kt0 = m0 / BK;                 // the stored A is zero above the diagonal"}[tri]
        all_fetch = lambda rs, k0: "".join(ld_piece_a(rs, p_, k0) for p_ in range(PA)) + "".join(ld_piece_b(rs, p_, k0) for p_ in range(PB))
        all_store = lambda rs, buf: "".join(st_piece_a(rs, p_, buf) for p_ in range(PA)) + "".join(st_piece_b(rs, p_, buf) for p_ in range(PB))
        kloop = f"""    {krange}
    float4 ra0[{PA}], rb0[{PB}], ra1[{PA}], rb1[{PB}];           // two sets of registers for tiles on their way to LDS
{frag_decl}    {{
{all_fetch(0, "kt0 * BK")}{all_store(0, "gb" if G > 1 else "0u")}{all_fetch(1, "min(kt0 + 1u, nk - 1u) * BK")}    }}
    __syncthreads();
    for (u32 kt = kt0; ; kt += 2u) {{
{deep_step(0, 0, 1, "min(kt + 2u, nk - 1u) * BK")}        __syncthreads();
        if (kt + 1u >= nk) break;
{deep_step(1, 1, 0, "min(kt + 3u, nk - 1u) * BK")}        __syncthreads();
        if (kt + 2u >= nk) break;"""
    split_head = split_tail = ""
    if splitk:
        split_head = """    const u32 kbeg = blockIdx.y * kchunk, kend = min(g.K, kbeg + kchunk);
    const u64 slab_elts = (u64)g.M * g.N;
    float* __restrict__ slab = W + ((u64)blockIdx.z * gridDim.y + blockIdx.y) * slab_elts;
"""
    if deep:
        loop_body = ""
    elif exact:
        # one straight run of code per k step: fetch, fence, MFMA run, LDS stores of what was fetched
        loop_body = f"""        load_tiles(min(kt + 1u, nk - 1u) * BK);
        __builtin_amdgcn_sched_barrier(0);
{mfma_run}
        stash_tiles(buf ^ 1u);
        __syncthreads();"""
    else:
        loop_body = f"""        if (kt + 1u < nk) load_tiles((kt + 1u) * BK);
{mfma_run}
        if (kt + 1u < nk) stash_tiles(buf ^ 1u);
        __syncthreads();"""
    group_head = group_join = ""
    if G > 1:
        group_head = "    const u32 kbeg = grp * kchunk, kend = min(g.K, kbeg + kchunk);            // this group's slice of k\n"
        group_join = f"""    // the groups' partial tiles meet in LDS (entry-major: a wavefront writes 64 consecutive floats); group 0 adds them in group order
    {f"float (*Red)[{MI * NJ * NE}][{T}] = reinterpret_cast<float (*)[{MI * NJ * NE}][{T}]>(&As[0][0][0]);      // (behind the last barrier of the k loop nobody reads the tiles any more)" if red_in_a else f"__shared__ float Red[{G - 1}][{MI * NJ * NE}][{T}];"}
    if (grp != 0u) {{
        #pragma unroll
        for (int i = 0; i < MI; ++i)
            #pragma unroll
            for (int j = 0; j < NJ; ++j)
                #pragma unroll
                for (int e = 0; e < {NE}; ++e) Red[grp - 1u][(i * NJ + j) * {NE} + e][tid] = acc[i][j][e];
    }}
    __syncthreads();
    if (grp != 0u) return;
    #pragma unroll
    for (int q = 0; q < {G - 1}; ++q)
        #pragma unroll
        for (int i = 0; i < MI; ++i)
            #pragma unroll
            for (int j = 0; j < NJ; ++j)
                #pragma unroll
                for (int e = 0; e < {NE}; ++e) acc[i][j][e] += Red[q][(i * NJ + j) * {NE} + e][tid];

"""
    f4v_typedef = "" if S == 32 else "\ntypedef float f4v __attribute__((ext_vector_type(4)));"
    src = f"""{PRELUDE}
typedef float f16v __attribute__((ext_vector_type(16)));{f4v_typedef}
struct f3v {{ float x, y, z; }};
struct MMArgs {{ u32 M, N, K, nbc, sa0, sa1, sb0, sb1; }};
#define BM {BM}u
#define BN {BN}u
#define BK {BK}u
#define MI {MI}
#define NJ {NJ}
#define KEND {"kend" if splitk or G > 1 else "g.K"}
extern "C" __global__ __launch_bounds__({G * T}) void {name}(const float* __restrict__ A,
        const float* __restrict__ B, float* __restrict__ C, MMArgs g{", const float* __restrict__ E" if epi else ""}{", const float* __restrict__ gain, float eps, float* __restrict__ yn, float* __restrict__ rinv" if norm else ""}{", float* __restrict__ W, u32 kchunk" if splitk else ""}{", u32 kchunk" if G > 1 else ""}) {{
    {decl_a}
    {decl_b}

    // ---- which C tile: XCD-contiguous renumbering, then groups of 8 tile rows
    const u32 tiles_m = (g.M + BM - 1u) / BM, tiles_n = (g.N + BN - 1u) / BN;
    const u32 nblk = tiles_m * tiles_n;
    u32 pid = blockIdx.x;
    if ((nblk & 7u) == 0u) pid = (pid & 7u) * (nblk >> 3) + (pid >> 3);
    const u32 width = 8u * tiles_n;
    const u32 first_m = (pid / width) * 8u;
    const u32 gsz = min(tiles_m - first_m, 8u);
    const u32 tm = first_m + (pid % width) % gsz, tn = (pid % width) / gsz;
{m0n0}
{skip_tile}
    const u32 zb = blockIdx.z / g.nbc, zc = blockIdx.z % g.nbc;
    A += (u64)zb * g.sa0 + (u64)zc * g.sa1;
    B += (u64)zb * g.sb0 + (u64)zc * g.sb1;
    C += (u64)blockIdx.z * g.M * g.N;
{split_head}
    {f"const u32 grp = threadIdx.x / {T}u, tid = threadIdx.x % {T}u" if G > 1 else "const u32 tid = threadIdx.x"}, lane = tid & 63u, wave = tid >> 6;
{group_head}    const u32 r = lane & {S - 1}u, h = lane >> {5 if S == 32 else 4};
    const u32 wm0 = (wave / {WN}u) * {S * MI}u, wn0 = (wave % {WN}u) * {S * NJ}u;
    {idx_a}
    {idx_b}

    {'f16v' if S == 32 else 'f4v'} acc[MI][NJ];
    #pragma unroll
    for (int i = 0; i < MI; ++i)
        #pragma unroll
        for (int j = 0; j < NJ; ++j)
            #pragma unroll
            for (int e = 0; e < {NE}; ++e) acc[i][j][e] = 0.f;

    float4 ra[{PA}], rb[{PB}];
    auto load_tiles = [&](u32 k0) {{
{load_a}{load_b}    }};
    auto stash_tiles = [&](u32 buf) {{
{stash_a}{stash_b}    }};

{kloop}
{loop_body}
    }}

{group_join}    #pragma unroll
    for (int i = 0; i < MI; ++i)
        #pragma unroll
        for (int e = 0; e < {NE}; ++e) {{
            const u32 row = {row_expr};
            if (row < g.M) {{
                float* __restrict__ crow = {"slab" if splitk else "C"} + (u64)row * g.N;
{store}
            }}
        }}
{split_tail}}}
"""
    if epi:
        assert epi in ("add", "relu", "gate", "bias") and not strided
        macro = {"add": "((cv) + (ev))", "relu": "((cv) > 0.0f ? (cv) : 0.0f)", "gate": "((ev) > 0.0f ? (cv) : 0.0f)",
                 "bias": "((cv) + (ev))"}[epi]
        edits = [("struct f3v {", f"#define EPI(cv, ev) {macro}\nstruct f3v {{")]
        if epi != "bias":                               # (a bias row is the same for every batch entry)
            edits.append(("C += (u64)blockIdx.z * g.M * g.N;", "C += (u64)blockIdx.z * g.M * g.N;\n    E += (u64)blockIdx.z * g.M * g.N;"))
        if tb:
            edits.append(("crow[col] = acc[i][j][e];", "crow[col] = EPI(acc[i][j][e], ev[i][j][e]);"))
        else:
            edits.append(("crow[col + j] = acc[i][j][e];", "crow[col + j] = EPI(acc[i][j][e], ev[i][j][e]);"))
            if vecb and NJ == 4:
                edits.append(("make_float4(acc[i][0][e], acc[i][1][e], acc[i][2][e], acc[i][3][e]);",
                              "make_float4(EPI(acc[i][0][e], ev[i][0][e]), EPI(acc[i][1][e], ev[i][1][e]), "
                              "EPI(acc[i][2][e], ev[i][2][e]), EPI(acc[i][3][e], ev[i][3][e]));"))
        if epi != "relu":
            # The entries of E this lane will need, fetched with clamped (always valid) addresses and no
            # branch, so that all loads are in flight together: ahead of the k loop where they fit in few
            # registers, right after it otherwise.
            if tb:
                fetch = ("#pragma unroll\n            for (int j = 0; j < NJ; ++j) "
                         f"ev[i][j][e] = erow[min(n0 + wn0 + {S}u * j + r, g.N - 1u)];")
            elif vecb and NJ == 4:                     # vecb vouches for 16-byte alignment of E as of C, and N % 4 == 0
                fetch = ("const float4 q = *reinterpret_cast<const float4*>(erow + min(n0 + wn0 + 4u * r, g.N - 4u));\n"
                         "            ev[i][0][e] = q.x; ev[i][1][e] = q.y; ev[i][2][e] = q.z; ev[i][3][e] = q.w;")
            else:
                fetch = (f"#pragma unroll\n            for (int j = 0; j < NJ; ++j) "
                         f"ev[i][j][e] = erow[min(n0 + wn0 + {NJ}u * r + j, g.N - 1u)];")
            pre = f"""    float ev[MI][NJ][{NE}];
    #pragma unroll
    for (int i = 0; i < MI; ++i)
        #pragma unroll
        for (int e = 0; e < {NE}; ++e) {{
            const float* __restrict__ erow = {'E' if epi == 'bias' else f'E + (u64)min({row_expr}, g.M - 1u) * g.N'};
            {fetch}
        }}

"""
            anchor = "    float4 ra[" if MI * NJ * NE <= 32 else f"    #pragma unroll\n    for (int i = 0; i < MI; ++i)\n        #pragma unroll\n        for (int e = 0; e < {NE}; ++e) {{\n            const u32 row"
            edits.append((anchor, pre + anchor))
        else:
            edits.append(("ev[i][", "acc[i]["))         # relu looks at the result only
        for was, now in edits:
            assert src.count(was) >= 1, was
            src = src.replace(was, now)
        return src, name, _fmt("P", "P", "P", "8I", "P", *(("P", "f", "P", "P") if norm else ()))
    if strided:
        for was, now in (("struct MMArgs { u32 M, N, K, nbc, sa0, sa1, sb0, sb1; };",
                          "struct MMArgs { u32 M, N, K, nbc, sa0, sa1, sb0, sb1, lda, ldb, ldc, sc0, sc1; };"),
                         ("A + (u64)k * g.M + col" if ta else "A + (u64)row * g.K + k",
                          "A + (u64)k * g.lda + col" if ta else "A + (u64)row * g.lda + k"),
                         ("B + (u64)row * g.K + k" if tb else "B + (u64)k * g.N + col",
                          "B + (u64)row * g.ldb + k" if tb else "B + (u64)k * g.ldb + col"),
                         ("C += (u64)blockIdx.z * g.M * g.N;", "C += (u64)zb * g.sc0 + (u64)zc * g.sc1;"),
                         ("C + (u64)row * g.N;", "C + (u64)row * g.ldc;")):
            assert src.count(was) >= 1, was                       # (the deep form names each operand address once per fetch pass)
            src = src.replace(was, now)
        return src, name, _fmt("P", "P", "P", "13I")
    return src, name, _fmt("P", "P", "P", "8I", *(("P", "f", "P", "P") if norm else ()), *(("P", "I") if splitk else ()), *(("I",) if G > 1 else ()))


@cache
def matmul_pair_kernel(first: tuple, second: tuple) -> tuple[str, str, str]:
    """Two independent products in one launch: the blocks of `first` followed by the blocks of `second`,
    each given as the argument tuple of matmul_kernel (tile, access widths, transposed forms, epilogue).

    The backward pass of a linear layer is such a pair -- dX = G W and dW = G^T X share G and nothing
    else -- and each of them alone leaves most of the chip idle for the few microseconds a short k loop
    takes; launched together they overlap.  The two bodies are the product kernels themselves, compiled as
    device functions in namespaces of their own and called with the block index they would have had
    (x = b % tiles, z = b / tiles), so every output element is computed by the same instructions in the
    same order as in a launch of its own: same bits.  Both bodies stage their operands in one LDS
    buffer sized for the larger; the block has the thread count of the larger body, and the wavefronts
    the smaller one does not use leave at once (a barrier waits only for the wavefronts still running).
    Arguments: those of the first product (A, B, C, its sizes and strides, E if it has an epilogue), those
    of the second, then the number of blocks of the first and the tile counts per batch entry of both."""
    import re
    parts = []
    for tag, a in (("p0", first), ("p1", second)):
        WM, WN, MI, NJ, BK, veca, vecb, ta, tb, tri, strided, epi, S, *rest = a
        exact, deep = bool(rest and rest[0]), bool(len(rest) > 1 and rest[1])
        assert not tri and not strided
        src, name, fmt = matmul_kernel(WM, WN, MI, NJ, BK, veca, vecb, ta, tb, tri, strided, epi, S, False, False, exact, 1, deep)
        assert src.startswith(PRELUDE)
        body = src[len(PRELUDE):]
        body, n = re.subn(r'extern "C" __global__ __launch_bounds__\(\d+\) void \w+\(',
                          "static __device__ __forceinline__ void body(const u32 bid_x, const u32 bid_z, float* __restrict__ lds, ", body)
        assert n == 1
        assert "blockIdx.y" not in body
        body = body.replace("blockIdx.x", "bid_x").replace("blockIdx.z", "bid_z")
        decls = re.findall(r"__shared__ __attribute__\(\(aligned\(16\)\)\) float (\w+)\[2\]\[(\d+)\]\[(\d+)\];", body)
        assert [d[0] for d in decls] == ["As", "Bs"], decls
        at = 0
        for nm, r_, c_ in decls:
            body = body.replace(f"__shared__ __attribute__((aligned(16))) float {nm}[2][{r_}][{c_}];",
                                f"float (*{nm})[{r_}][{c_}] = reinterpret_cast<float (*)[{r_}][{c_}]>(lds + {at}u);")
            at += 2 * int(r_) * int(c_)
        assert 4 * at == matmul_lds_bytes(WM, WN, MI, NJ, BK, ta, tb, S)
        parts.append({"tag": tag, "name": name, "body": body, "threads": 64 * WM * WN, "lds": at, "epi": bool(epi), "fmt": fmt})
    threads = max(p["threads"] for p in parts)
    lds = max(p["lds"] for p in parts)
    assert 4 * lds <= MATMUL_LDS_LIMIT
    name = "pair_" + parts[0]["name"].replace("matmul_", "") + "__" + parts[1]["name"].replace("matmul_", "")
    undef = "#undef BM\n#undef BN\n#undef BK\n#undef MI\n#undef NJ\n#undef EPI\n"
    src = PRELUDE
    params, calls = [], []
    for i, p in enumerate(parts):
        src += f"namespace {p['tag']} {{\n{p['body']}}}\n{undef}"
        params.append(f"const float* __restrict__ A{i}, const float* __restrict__ B{i}, float* __restrict__ C{i}, {p['tag']}::MMArgs g{i}"
                      + (f", const float* __restrict__ E{i}" if p["epi"] else ""))
        calls.append(f"{p['tag']}::body(b % tiles{i}, b / tiles{i}, lds, A{i}, B{i}, C{i}, g{i}" + (f", E{i}" if p["epi"] else "") + ");")
    src += f"""
extern "C" __global__ __launch_bounds__({threads}) void {name}({params[0]},
        {params[1]}, u32 nblk0, u32 tiles0, u32 tiles1) {{
    __shared__ __attribute__((aligned(16))) float lds[{lds}];
    if (blockIdx.x < nblk0) {{
        if (threadIdx.x >= {parts[0]['threads']}u) return;
        const u32 b = blockIdx.x;
        {calls[0]}
    }} else {{
        if (threadIdx.x >= {parts[1]['threads']}u) return;
        const u32 b = blockIdx.x - nblk0;
        {calls[1]}
    }}
}}
"""
    return src, name, "@" + parts[0]["fmt"][1:] + parts[1]["fmt"][1:] + "III"


# name -> (WM, WN, MI, NJ, BK): block tile = (32*MI*WM) x (32*NJ*WN), 64*WM*WN threads.
# Kept after sweeps on MI355X (TFLOP/s at 4096^3 / 8192x768x768 / batch 8 of 768x3072x1024):
#   256x256 (8 waves, 128 acc regs)   136 /  .. /  ..    largest problems, one block per CU
#   256x128 (4 waves, 128 acc regs)   135
#   128x256 (8 waves,  64 acc regs)   129
#   128x128 (4 waves of 64x64)        128 /  68 / 107
#   192x192 (4 waves of 96x96)         .. /  .. / 124    N or M a multiple of 192 (768, 3072)
#   128x192 (8 waves of 32x96)         .. / 100 / 114    8192x768 as exactly 256 blocks
#   128x96, 128x64 (4 waves of 32xBN)  .. / 103, 107     narrow outputs: 2-3 resident blocks per CU
# Every tile accumulates k in the same order, so the choice never changes a result bit.
MATMUL_CONFIGS = {
    "256x256": (4, 2, 2, 4, 16),
    "256x256k32": (4, 2, 2, 4, 32),     # the same tiles with k walked 32 at a time: half the barriers, one block per CU
    "256x128": (4, 1, 2, 4, 16),
    "256x128k32": (4, 1, 2, 4, 32),
    "128x256": (4, 2, 1, 4, 32),
    "192x192": (2, 2, 3, 3, 16),
    "128x192": (4, 2, 1, 3, 32),
    "128x128": (2, 2, 2, 2, 32),
    "128x96": (4, 1, 1, 3, 32),
    "128x64": (4, 1, 1, 2, 32),
    "128x128w16": (4, 4, 1, 1, 32),     # sixteen waves of 32x32: outputs of about 256 tiles (2048^2), where a CU holds
    "128x64w8": (4, 2, 1, 1, 32),       # one block and only its own waves can overlap loads with MFMA (2048^3: 115
    "64x128w8": (2, 4, 1, 1, 32),       # against 97 TFLOP/s for four waves of 64x64); the eight-wave halves for narrow outputs
    "64x64": (2, 2, 1, 1, 16),
    "64x64k32": (2, 2, 1, 1, 32),
    "64x64k64": (2, 2, 1, 1, 64),       # same tile, K walked 64 at a time: fewer barriers when one block per CU
    "32x32": (1, 1, 1, 1, 16),          # has nobody to overlap with (1024^3: 73 against 62 TFLOP/s)
    # sixth entry 16: wavefronts of 16x16 (v_mfma_f32_16x16x4_f32) for small outputs with a long k, where the
    # chain of MFMA steps per wavefront is what takes the time (2048 x 128 x 512)
    "64x64m16": (4, 4, 1, 1, 64, 16),
    "64x32m16": (4, 2, 1, 1, 32, 16),
    "32x32m16": (2, 2, 1, 1, 32, 16),
    # the same with k walked 128 at a time: a product with k = 128 is then one round of loads (all in flight
    # together), one barrier and one run of MFMA steps instead of four dependent rounds
    "64x64m16k128": (4, 4, 1, 1, 128, 16),
    "32x32m16k128": (2, 2, 1, 1, 128, 16),
    "32x32m16k64": (2, 2, 1, 1, 64, 16),
}
MATMUL_SMALL_TILES = ("64x64", "64x64k32", "64x64k64", "32x32", "64x64m16", "64x32m16", "32x32m16", "64x64m16k128", "32x32m16k128", "32x32m16k64")


def matmul_tile_shape(tile: str) -> tuple[int, int, int]:
    """(rows, columns, threads) of a block of the named configuration."""
    wm, wn, mi, nj, _, *s = MATMUL_CONFIGS[tile]
    edge = s[0] if s else 32
    return edge * mi * wm, edge * nj * wn, 64 * wm * wn


# (relative per-CU throughput when the chip is full, resident blocks per CU): the model that
# picks a tile for a shape nobody has timed
MATMUL_TILE_MODEL = {
    "256x256": (1.00, 1), "256x128": (0.99, 2), "128x256": (0.95, 1), "192x192": (0.93, 2), "128x192": (0.88, 1),
    "128x128": (0.94, 2), "128x128w16": (0.86, 1), "128x96": (0.86, 3), "128x64": (0.85, 4), "64x64": (0.74, 8), "32x32": (0.60, 8),
}


# =====================================================================================
# one row times a transposed matrix (decoding)
# =====================================================================================

@cache
def row_matmul_nt_kernel(epi: str = "", norm_nval: int = 0, kv: bool = False) -> tuple[str, str, str]:
    """y[n] = sum_k x[k] * W[n][k] for one row x (K) and W stored (N, K): the linear layers of a
    decoding step, where an MFMA tile would hold one useful row in 16.  One wavefront per output:
    lane l multiplies the 16-byte items l, l + 64, ... of the row of W with the same items of x
    (K % 4 == 0, 16-byte aligned rows), four independent loads in flight, and the 64 partial sums are
    added across the wavefront.  epi as in matmul_kernel ("add": + e[n], "relu", "gate": e[n] > 0).
    norm_nval > 0: x is first RMS-normalised with the gain row g -- (x * r) * g with
    r = 1 / sqrt(sum(x^2) / K + eps) -- by every wavefront for itself, the row (at most 64 * norm_nval
    items) in registers: the statements of rmsnorm_fwd_kernel, so the values that enter the product
    are the ones that kernel would have stored, and the launch between the two disappears.
    kv (no epilogue): W is the stacked q, k, v projection (N = 3 * C3).  The first third of the outputs goes
    to y as usual; the second and third are the new position's key and value and go straight to row
    (int)slot[0] of the (rows, C3) stores kc and vc (nothing is stored for a row outside [0, rows), as
    row_store_kernel has it): the launch that copied them there disappears.  Arguments after the others:
    kc, vc, slot, C3, rows."""
    assert epi in ("", "add", "relu", "gate") and not (kv and epi)
    name = f"row_matmul_nt{'_' + epi if epi else ''}{f'_rms{norm_nval}' if norm_nval else ''}{'_kv' if kv else ''}"
    fin = {"": "acc", "add": "acc + e[n]", "relu": "(acc > 0.0f ? acc : 0.0f)", "gate": "(e[n] > 0.0f ? acc : 0.0f)"}[epi]
    if norm_nval:
        comps = (".x", ".y", ".z", ".w")
        sq = " + ".join(f"v[k]{c} * v[k]{c}" for c in comps)
        outs = "".join(f"            o{c} = (v[k]{c} * r) * g{c};\n" for c in comps)
        body = f"""    float4 v[{norm_nval}];
    float ss = 0.0f;
    #pragma unroll
    for (u32 k = 0; k < {norm_nval}u; ++k) {{
        const u32 c = lane + k * 64u;
        if (c < K4) {{ v[k] = x4[c]; ss += {sq}; }}
    }}
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / (float)K + eps);
    const float4* __restrict__ wv = reinterpret_cast<const float4*>(gain);
    float acc = 0.0f;
    #pragma unroll
    for (u32 k = 0; k < {norm_nval}u; ++k) {{
        const u32 c = lane + k * 64u;
        if (c < K4) {{
            const float4 g = wv[c];
            float4 o;
{outs}            acc = dot4(w4[c], o, acc);
        }}
    }}
"""
        extra, fmt = ", const float* __restrict__ gain, float eps", _fmt("P", "P", "P", "P", "I", "I", "P", "f")
    else:
        body = """    float acc = 0.0f;
    u32 c = lane;
    for (; c + 192u < K4; c += 256u) {
        const float4 a0 = w4[c], a1 = w4[c + 64u], a2 = w4[c + 128u], a3 = w4[c + 192u];
        const float4 b0 = x4[c], b1 = x4[c + 64u], b2 = x4[c + 128u], b3 = x4[c + 192u];
        acc = dot4(a0, b0, acc); acc = dot4(a1, b1, acc); acc = dot4(a2, b2, acc); acc = dot4(a3, b3, acc);
    }
    for (; c < K4; c += 64u) acc = dot4(w4[c], x4[c], acc);
"""
        extra, fmt = "", _fmt("P", "P", "P", "P", "I", "I")
    store = f"if (lane == 0u) y[n] = {fin};"
    if kv:
        extra += ", float* __restrict__ kc, float* __restrict__ vc, const float* __restrict__ slot, u32 C3, u32 rows"
        fmt += "PPPII"
        store = """if (lane == 0u) {
        if (n < C3) y[n] = acc;
        else {
            const float fi = slot[0];
            if (fi >= 0.0f && fi < (float)rows) {
                const u32 third = n / C3;
                (third == 1u ? kc : vc)[(u64)(u32)fi * C3 + (n - third * C3)] = acc;
            }
        }
    }"""
    src = f"""{PRELUDE}
static __device__ __forceinline__ float dot4(float4 a, float4 b, float acc) {{
    acc = fmaf(a.x, b.x, acc); acc = fmaf(a.y, b.y, acc); acc = fmaf(a.z, b.z, acc); return fmaf(a.w, b.w, acc);
}}
extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ x,
        const float* __restrict__ W, float* __restrict__ y, const float* __restrict__ e, u32 N, u32 K{extra}) {{
    const u32 lane = threadIdx.x & 63u, n = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (n >= N) return;
    const u32 K4 = K >> 2;
    const float4* __restrict__ w4 = reinterpret_cast<const float4*>(W + (u64)n * K);
    const float4* __restrict__ x4 = reinterpret_cast<const float4*>(x);
{body}    acc = wave_sum(acc);
    {store}
}}
"""
    return src, name, fmt


# =====================================================================================
# the ends of a decoding step: embedding of the token(s) to feed, choice of the next one
# =====================================================================================

@cache
def decode_embed_kernel(window: bool) -> tuple[str, str, str]:
    """The input of a decoding step, from device-resident state, in one launch.
    window = False: x[0, :] = wte[tok] + wpe[pos] for the token tok[0] fed at index s = slot[0], with
      pos = s, or s + clamp(s, 0, 1) when refpos (the reference numbers an incremental token one too
      high, examples/gpt.py:199), and hidden[j] = (j > s) for the T cache rows: what the clamp, the add,
      the comparison with arange, the two gathers and the add of the op-by-op step compute.
    window = True: x[t, :] = wte[seq[s - (T - 1) + t]] + wpe[t] for t < T: the window of the last T
      tokens out of the token buffer (rows, 1), embedded at positions 0 .. T - 1.
    Rows are looked up as embedding_kernel does it -- offset (int)(id * W) formed in float, a row that
    does not lie inside its table reads as zeros -- and the sum is the one fp32 addition of the add
    kernel.  One wavefront per position."""
    name = "decode_embed_window" if window else "decode_embed"
    if window:
        head = """    const u32 t = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (t >= T) return;
    const float w = (float)t + (slot[0] - (float)(T - 1u));   // arange + (slot - (T - 1)), as the op-by-op step forms it
    const int si = (int)(w * 1.0f);                             // the token buffer is a table of rows of one float
    const float tok = (si < 0 || (u64)si + 1u > (u64)rows) ? 0.0f : seq[si];
    const float pos = (float)t;
    float* __restrict__ dst = x + (u64)t * C;
"""
        params = "const float* __restrict__ seq, const float* __restrict__ slot, float* __restrict__ x, u32 C, u32 V, u32 P, u32 T, u32 rows"
        fmt = _fmt("P", "P", "P", "P", "P", "I", "I", "I", "I", "I")
        tail = ""
    else:
        head = """    if (blockIdx.x != 0u || threadIdx.x >= 64u) {              // the other wavefronts write the mask of the cache rows
        const u32 j = blockIdx.x * 256u + threadIdx.x - 64u;
        if (j < T) hidden[j] = (float)j > slot[0] ? 1.0f : 0.0f;
        return;
    }
    const float s = slot[0];
    const float tok = tokp[0];
    const float pos = refpos ? s + fminf(fmaxf(s, 0.0f), 1.0f) : s;
    float* __restrict__ dst = x;
"""
        params = ("const float* __restrict__ tokp, const float* __restrict__ slot, float* __restrict__ x, float* __restrict__ hidden, "
                  "u32 C, u32 V, u32 P, u32 T, u32 refpos")
        fmt = _fmt("P", "P", "P", "P", "P", "P", "I", "I", "I", "I", "I")
        tail = ""
    src = f"""{PRELUDE}
extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ wte, const float* __restrict__ wpe,
        {params}) {{
    const u32 lane = threadIdx.x & 63u;
{head}    const int ti = (int)(tok * (float)C), pi = (int)(pos * (float)C);
    const bool tok_ok = ti >= 0 && (u64)ti + C <= (u64)V * C, pos_ok = pi >= 0 && (u64)pi + C <= (u64)P * C;
    for (u32 j = lane; j < C; j += 64u)
        dst[j] = (tok_ok ? wte[(long long)ti + j] : 0.0f) + (pos_ok ? wpe[(long long)pi + j] : 0.0f);
{tail}}}
"""
    return src, name, fmt


@cache
def decode_next_kernel() -> tuple[str, str, str]:
    """The end of a decoding step in one launch: next = index of the first maximum of the V logits
    (argmax_kernel's rule: strict '>' from (-FLT_MAX, 0)), then seq[s + 1] = next for s = slot[0] (skipped
    when s + 1 lies outside the (rows, 1) token buffer), tok[0] = next and slot[0] = s + 1 -- what argmax,
    add, row_store and two copies do in the op-by-op step.  One block."""
    name = "decode_next"
    src = f"""{PRELUDE}{_ARGMAX_PAIR}
extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ logits, float* __restrict__ tok,
        float* __restrict__ slot, float* __restrict__ seq, u32 V, u32 rows) {{
    __shared__ float sv[4];
    __shared__ u32 si[4];
    float best = NEG_FLT_MAX;
    u32 bi = 0u;
    for (u32 j = threadIdx.x; j < V; j += 256u) {{ const float v = logits[j]; if (v > best) {{ best = v; bi = j; }} }}
    wave_argmax(best, bi);
    if ((threadIdx.x & 63u) == 0u) {{ sv[threadIdx.x >> 6] = best; si[threadIdx.x >> 6] = bi; }}
    __syncthreads();
    if (threadIdx.x == 0u) {{
        #pragma unroll
        for (u32 w = 1; w < 4u; ++w) {{ const float ov = sv[w]; const u32 oi = si[w]; TAKE(best, bi, ov, oi) }}
        const float nxt = (float)bi, ns = slot[0] + 1.0f;
        if (ns >= 0.0f && ns < (float)rows) seq[(u32)ns] = nxt;
        tok[0] = nxt;
        slot[0] = ns;
    }}
}}
"""
    return src, name, _fmt("P", "P", "P", "P", "I", "I")


@cache
def decode_sample_kernel() -> tuple[str, str, str]:
    """The end of a *sampling* decoding step in one launch: the next token is drawn from
    softmax(logits / temperature) by inversion, as np.random.choice(V, p=probs) draws it
    (examples/gpt.py:215-221, :259-260): next = the first index whose running sum of the
    probabilities exceeds the uniform number.  The uniform number is u[s] for s = slot[0], the
    index of the token just fed -- a device array filled beforehand, so a captured step draws a
    new number on every replay.  Then, as decode_next: seq[s + 1] = next (skipped outside the
    (rows, 1) token buffer), tok[0] = next, slot[0] = s + 1.

    One block.  Thread t owns the contiguous run [t * ceil(V / 256), ...) of the vocabulary:
    e_j = exp(x_j / temperature - max) is summed over the run in index order, the runs are joined
    by a scan over the 256 threads, and the thread whose run contains the target u * total walks
    it again to find the index.  The sums are fp32 in a fixed order: the same logits and the
    same u always give the same token.  If rounding leaves u * total at or above every running
    sum, the last index of non-zero probability is taken."""
    name = "decode_sample"
    src = f"""{PRELUDE}
extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ logits, const float* __restrict__ u,
        float* __restrict__ tok, float* __restrict__ slot, float* __restrict__ seq, u32 V, u32 rows, u32 n_u,
        float temperature) {{
    __shared__ float swave[4];
    __shared__ float sruns[4];
    __shared__ u32 sfound[4];
    const u32 t = threadIdx.x, lane = t & 63u, w = t >> 6;
    const u32 run = (V + 255u) / 256u;
    const u32 j0 = min(t * run, V), j1 = min(j0 + run, V);
    float m = NEG_FLT_MAX;
    for (u32 j = j0; j < j1; ++j) m = fmaxf(m, logits[j] / temperature);
    m = wave_max(m);
    if (lane == 0u) swave[w] = m;
    __syncthreads();
    m = fmaxf(fmaxf(swave[0], swave[1]), fmaxf(swave[2], swave[3]));
    float own = 0.0f;
    for (u32 j = j0; j < j1; ++j) own += expf(logits[j] / temperature - m);
    float upto = own;                                   // inclusive scan over the lanes of the wavefront
    #pragma unroll
    for (u32 d = 1; d < 64u; d <<= 1) {{
        const float o = __shfl_up(upto, d, WAVE);
        if (lane >= d) upto += o;
    }}
    if (lane == 63u) sruns[w] = upto;
    __syncthreads();
    float before = 0.0f;
    for (u32 k = 0; k < w; ++k) before += sruns[k];
    const float total = ((sruns[0] + sruns[1]) + sruns[2]) + sruns[3];
    const float sf = slot[0];
    const u32 ui = (sf >= 0.0f && sf < (float)n_u) ? (u32)sf : 0u;
    const float target = u[ui] * total;
    float sum = before + (upto - own);                  // everything in front of this thread's run
    u32 found = V;
    for (u32 j = j0; j < j1; ++j) {{
        sum += expf(logits[j] / temperature - m);
        if (sum > target) {{ found = j; break; }}
    }}
    #pragma unroll
    for (u32 d = 32; d >= 1u; d >>= 1) found = min(found, (u32)__shfl_xor((int)found, (int)d, WAVE));
    if (lane == 0u) sfound[w] = found;
    __syncthreads();
    if (t == 0u) {{
        found = min(min(sfound[0], sfound[1]), min(sfound[2], sfound[3]));
        if (found >= V) {{                               // rounding left the target beyond every running sum: the last token that can be drawn
            found = V - 1u;
            while (found > 0u && !(expf(logits[found] / temperature - m) > 0.0f)) --found;
        }}
        const float nxt = (float)found, ns = sf + 1.0f;
        if (ns >= 0.0f && ns < (float)rows) seq[(u32)ns] = nxt;
        tok[0] = nxt;
        slot[0] = ns;
    }}
}}
"""
    return src, name, _fmt("P", "P", "P", "P", "P", "I", "I", "I", "f")


# =====================================================================================
# attention for one new position (decoding)
# =====================================================================================

DECODE_ATTENTION_MAX_N = 1024
DECODE_ATTENTION_MAX_D = 64


@cache
def decode_attention_kernel(npl: int, masked: bool, vec: int) -> tuple[str, str, str]:
    """softmax(q k^T * scale) v for one query position per (sequence, head) against n cached positions:
    the three launches of the decoding branch of examples/gpt.py:58-63 (scores, softmax, context) as one.
    One wavefront per (sequence, head).  q is (B, 1, C) with the head's d <= 64 values at b*C + head*d;
    the stores are (rows, B, C), row r of this head at r*pitch + b*C + head*d.  Lane l scores the
    positions l, l + 64, ... (npl of them at most, so n <= 64*npl): d multiply-adds each, times
    scale, -inf where `hidden` says so; maximum, exponentials and their sum are reduced over the
    wavefront; the probabilities pass through LDS.
    vec=4 (d in 4, 8, .. 64 a power of two, 16-byte aligned rows): key rows are read 16 bytes at a
    time, eight loads in flight; for the context the lanes form d/4 column groups times 256/d position
    groups, each lane adds p[r] * v[r][4 floats] over its share of the positions with sixteen loads in
    flight, and the position groups are joined by lane exchanges.
    vec=1: any d; lane j adds p[r] * v[r][j] over the positions (two interleaved halves when d <= 32)."""
    assert npl in (2, 4, 8, 16) and vec in (1, 4)
    name = f"decode_attention_r{npl}{'_m' if masked else ''}_v{vec}"
    if vec == 4:
        dot = """                const float4* __restrict__ kr = reinterpret_cast<const float4*>(kh + (u64)pos * pitch);
                for (u32 j0 = 0; j0 < d4; j0 += 8u) {
                    float4 kv[8];
                    #pragma unroll
                    for (u32 t = 0; t < 8u; ++t) kv[t] = kr[min(j0 + t, d4 - 1u)];
                    #pragma unroll
                    for (u32 t = 0; t < 8u; ++t) if (j0 + t < d4) {
                        const u32 j = 4u * (j0 + t);
                        acc = fmaf(qs[j], kv[t].x, acc); acc = fmaf(qs[j + 1u], kv[t].y, acc);
                        acc = fmaf(qs[j + 2u], kv[t].z, acc); acc = fmaf(qs[j + 3u], kv[t].w, acc);
                    }
                }"""
        context = """    const u32 CG = d4, PG = 64u / CG, cg = lane % CG;
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    #pragma unroll 16
    for (u32 pos = lane / CG; pos < n; pos += PG) {
        const float w = ps[pos];
        const float4 t = reinterpret_cast<const float4*>(vh + (u64)pos * pitch)[cg];
        o.x = fmaf(w, t.x, o.x); o.y = fmaf(w, t.y, o.y); o.z = fmaf(w, t.z, o.z); o.w = fmaf(w, t.w, o.w);
    }
    for (u32 off = CG; off < 64u; off <<= 1) {
        o.x += __shfl_xor(o.x, off, WAVE); o.y += __shfl_xor(o.y, off, WAVE);
        o.z += __shfl_xor(o.z, off, WAVE); o.w += __shfl_xor(o.w, off, WAVE);
    }
    if (lane < CG) reinterpret_cast<float4*>(y + at)[lane] = o;"""
    else:
        dot = """                const float* __restrict__ kr = kh + (u64)pos * pitch;
                for (u32 j0 = 0; j0 < d; j0 += 8u) {
                    float kv[8];
                    #pragma unroll
                    for (u32 t = 0; t < 8u; ++t) kv[t] = kr[min(j0 + t, d - 1u)];
                    #pragma unroll
                    for (u32 t = 0; t < 8u; ++t) if (j0 + t < d) acc = fmaf(qs[j0 + t], kv[t], acc);
                }"""
        context = """    const u32 W = d <= 32u ? 32u : 64u, step = 64u / W, j = lane % W;
    float o = 0.0f;
    if (j < d) {
        #pragma unroll 16
        for (u32 pos = lane / W; pos < n; pos += step) o = fmaf(ps[pos], vh[(u64)pos * pitch + j], o);
    }
    if (step == 2u) o += __shfl_xor(o, 32, WAVE);
    if (lane < d) y[at + lane] = o;"""
    hid = "if (hidden[pos] > 0.0f) acc = -__builtin_inff();" if masked else ""
    src = f"""{PRELUDE}
extern "C" __global__ __launch_bounds__(64) void {name}(const float* __restrict__ q,
        const float* __restrict__ ks, const float* __restrict__ vs, const float* __restrict__ hidden,
        float* __restrict__ y, u32 n, u32 C, u32 d, u32 pitch, u32 n_head, float scale) {{
    __shared__ float qs[{DECODE_ATTENTION_MAX_D}];
    __shared__ float ps[{64 * npl}];
    const u32 lane = threadIdx.x, b = blockIdx.x / n_head, at = b * C + (blockIdx.x % n_head) * d;
    const u32 d4 = d >> 2; (void)d4;
    const float* __restrict__ kh = ks + at;
    const float* __restrict__ vh = vs + at;
    if (lane < d) qs[lane] = q[at + lane];
    __syncthreads();
    float sc[{npl}];
    float m = -__builtin_inff();
    #pragma unroll
    for (u32 k = 0; k < {npl}u; ++k) {{
        const u32 pos = lane + 64u * k;
        float acc = -__builtin_inff();
        if (pos < n) {{
            acc = 0.0f;
{dot}
            acc *= scale;
            {hid}
        }}
        sc[k] = acc;
        m = fmaxf(m, acc);
    }}
    m = wave_max(m);
    float sum = 0.0f;
    #pragma unroll
    for (u32 k = 0; k < {npl}u; ++k) {{ sc[k] = expf(sc[k] - m); sum += sc[k]; }}
    sum = wave_sum(sum);
    #pragma unroll
    for (u32 k = 0; k < {npl}u; ++k) ps[lane + 64u * k] = sc[k] / sum;
    __syncthreads();
{context}
}}
"""
    return src, name, _fmt("P", "P", "P", "P", "P", "I", "I", "I", "I", "I", "f")


# =====================================================================================
# optimizer
# =====================================================================================

ATTN_SMALL_T = 128         # longest sequence, and
ATTN_SMALL_D = 32          # widest head, that the one-launch attention kernels hold in LDS


@cache
def attention_small_kernel(stage: str) -> tuple[str, str, str]:
    """Causal self-attention with the scores never leaving the chip (examples/gpt.py:50-55 run it as
    product, scale, mask, softmax, product; here for T <= 128 and a head width d <= 32 with
    d % 4 == 0, the char-GPT shapes): one launch forward, one backward.

    The heads are read where they lie inside (B, T, pitch) tensors -- row pitch `pitch`, batch stride
    T * pitch, head stride d -- zero-padded in LDS (row pitch 33).  The T x T score matrix of a head
    is cut into 32 x 32 tiles; only the tiles (ti, tj <= ti) on or below the diagonal are ever
    computed, the others are exact zeros.  One block of 8 wavefronts per (sequence, head, tile row
    i); grid = B * n_head * ceil(T / 32).  All products are 32 x 32 x 32 tile products on
    v_mfma_f32_32x32x2_f32 (lane l feeds A[l % 32][l / 32] and B[l / 32][l % 32] of a step; accumulator
    e of a lane is row 8 (e / 4) + 4 (l / 32) + e % 4, column l % 32), one wavefront per tile; partial
    tiles of one output are handed over through LDS and added in ascending tile order.

      "fwd"  block i: S(i, j) = q_i k_j^T * scale for j <= i, -inf above the diagonal -> LDS; row
             softmax, a wavefront per row (max, exp once, sum, divide); the probabilities go to
             p (B, n_head, T, T), zeros above the diagonal, for the backward pass; y_i = sum_j P(i, j) v_j
             goes to the (B, T, y_pitch) context in place.
      "bwd"  block i owns dq_i, dk_i and dv_i, so it needs dS(i, j <= i) and dS(t >= i, i): four tiles at
             most, a wavefront each.  delta = rowsum(dy * y) (equal to rowsum(dP * P), since y = P v);
             per tile dP = dy v^T and dS = P * (dP - delta) * scale; dq_i = sum_j dS(i, j) k_j;
             dk_i = sum_t dS(t, i)^T q_t; dv_i = sum_t P(t, i)^T dy_t (four more wavefronts, P read
             from memory in operand layout).  The gradients go into (B, T, g_pitch) tensors in place.
    Same mathematics as the chain of kernels, other order of additions inside the dot products."""
    assert stage in ("fwd", "bwd")
    name = f"attention_small_{stage}"
    common = r"""
typedef float f16v __attribute__((ext_vector_type(16)));
#define DP 33u                       /* LDS row pitch of the operand tiles (32 columns) */
#define SP 129u                      /* LDS row pitch of a tile row of scores (128 columns) */
#define TILE (32u * DP)
#define MFMA(a, b, c) __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0)
#define ZERO16(a) { _Pragma("unroll") for (int z_ = 0; z_ < 16; ++z_) a[z_] = 0.0f; }
// item `it` of a head's rows [row0, row0 + ..): row row0 + it / 8, columns 4 (it % 8) ..; zeros outside [0, T) x [0, d)
static __device__ __forceinline__ float4 head_part(const float* __restrict__ src, u32 it, u32 row0, u32 T, u32 d, u32 pitch) {
    const u32 row = row0 + (it >> 3), c4 = (it & 7u) << 2;
    return (row < T && c4 < d) ? *reinterpret_cast<const float4*>(src + (u64)row * pitch + c4) : make_float4(0.f, 0.f, 0.f, 0.f);
}
static __device__ __forceinline__ void put_part(float* __restrict__ dst, u32 it, const float4 v) {     // dst: LDS row of item 0
    float* q = dst + (it >> 3) * DP + ((it & 7u) << 2);
    q[0] = v.x; q[1] = v.y; q[2] = v.z; q[3] = v.w;
}
// acc += A B over 32 steps of k with A[m][k] = a[m * am + k * ak] and B[k][n] = b[k * bk + n * bn]; operands fetched first
static __device__ __forceinline__ void tile_product(f16v& acc, const float* __restrict__ a, u32 am, u32 ak,
                                                    const float* __restrict__ b, u32 bk, u32 bn, u32 r, u32 h) {
    float av[16], bv[16];
    #pragma unroll
    for (u32 s = 0; s < 16u; ++s) { av[s] = a[r * am + (2u * s + h) * ak]; bv[s] = b[(2u * s + h) * bk + r * bn]; }
    #pragma unroll
    for (u32 s = 0; s < 16u; ++s) acc = MFMA(av[s], bv[s], acc);
}
// partial tiles change hands as [slot][e][lane]
static __device__ __forceinline__ void put_partial(float* __restrict__ box, u32 slot, const f16v& acc, u32 lane) {
    #pragma unroll
    for (u32 e = 0; e < 16u; ++e) box[(slot * 16u + e) * 64u + lane] = acc[e];
}
// accumulator entries 4 g .. 4 g + 3 (rows row0 + 8 g + 4 h ..) of the sum of slots [s0, s1) -> a head in global memory
static __device__ __forceinline__ void sum_and_store(float* __restrict__ dst, const float* __restrict__ box, u32 s0, u32 s1,
                                                     u32 g, u32 row0, u32 T, u32 d, u32 pitch, u32 lane) {
    const u32 r = lane & 31u, h = lane >> 5;
    float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (u32 sl = s0; sl < s1; ++sl) {
        #pragma unroll
        for (u32 c = 0; c < 4u; ++c) v[c] += box[(sl * 16u + 4u * g + c) * 64u + lane];
    }
    #pragma unroll
    for (u32 c = 0; c < 4u; ++c) {
        const u32 row = row0 + 8u * g + 4u * h + c;
        if (row < T && r < d) dst[(u64)row * pitch + r] = v[c];
    }
}
"""
    if stage == "fwd":
        body = r"""
extern "C" __global__ __launch_bounds__(512) void attention_small_fwd(const float* __restrict__ q,
        const float* __restrict__ k, const float* __restrict__ v, float* __restrict__ y, float* __restrict__ p,
        u32 T, u32 d, u32 pitch, u32 y_pitch, u32 n_head, u32 nt, float scale) {
    __shared__ float Qs[TILE], Ks[4u * TILE], Vs[4u * TILE], Ss[32u * SP], box[4u * 1024u];
    const u32 bh = blockIdx.x / nt, i = blockIdx.x % nt, b = bh / n_head, hd = bh % n_head;
    const u32 t = threadIdx.x, w = t >> 6, lane = t & 63u, r = lane & 31u, h = lane >> 5;
    const u64 in_off = (u64)b * T * pitch + (u64)hd * d;
    {
        const u32 n_kv = 256u * (i + 1u);                   // 16-byte items of the key and value rows this tile row sees
        const float4 q4 = t < 256u ? head_part(q + in_off, t, 32u * i, T, d, pitch) : make_float4(0.f, 0.f, 0.f, 0.f);
        float4 k4[2], v4[2];
        #pragma unroll
        for (u32 n = 0; n < 2u; ++n)
            if (t + 512u * n < n_kv) { k4[n] = head_part(k + in_off, t + 512u * n, 0u, T, d, pitch); v4[n] = head_part(v + in_off, t + 512u * n, 0u, T, d, pitch); }
        if (t < 256u) put_part(Qs, t, q4);
        #pragma unroll
        for (u32 n = 0; n < 2u; ++n)
            if (t + 512u * n < n_kv) { put_part(Ks, t + 512u * n, k4[n]); put_part(Vs, t + 512u * n, v4[n]); }
    }
    __syncthreads();
    if (w <= i) {                                           // S(i, w) = q_i k_w^T
        f16v acc; ZERO16(acc)
        tile_product(acc, Qs, DP, 1u, Ks + w * TILE, 1u, DP, r, h);
        #pragma unroll
        for (u32 e = 0; e < 16u; ++e) {
            const u32 lr = 8u * (e >> 2) + 4u * h + (e & 3u), col = 32u * w + r;
            Ss[lr * SP + col] = col > 32u * i + lr ? -__builtin_inff() : acc[e] * scale;
        }
    }
    __syncthreads();
    {   // softmax: wavefront w takes rows w, w + 8, .. of the tile row; a lane holds columns lane and lane + 64 of each.
        // Columns 0 .. row are live, the rest of the row is 0
        float* __restrict__ pout = p + (u64)bh * T * T;
        const bool wide = i >= 2u;                          // the rows reach beyond column 63
        float x0[4], x1[4], m[4], sum[4];
        #pragma unroll
        for (u32 c = 0; c < 4u; ++c) {
            const u32 lr = w + 8u * c, row = 32u * i + lr;
            x0[c] = lane <= row ? Ss[lr * SP + lane] : -__builtin_inff();
            x1[c] = (wide && lane + 64u <= row) ? Ss[lr * SP + lane + 64u] : -__builtin_inff();
        }
        #pragma unroll
        for (u32 c = 0; c < 4u; ++c) m[c] = wave_max(fmaxf(fmaxf(x0[c], x1[c]), NEG_FLT_MAX));
        #pragma unroll
        for (u32 c = 0; c < 4u; ++c) {
            const u32 row = 32u * i + w + 8u * c;
            x0[c] = lane <= row ? expf(x0[c] - m[c]) : 0.0f;
            x1[c] = (wide && lane + 64u <= row) ? expf(x1[c] - m[c]) : 0.0f;
        }
        #pragma unroll
        for (u32 c = 0; c < 4u; ++c) sum[c] = wave_sum(x0[c] + x1[c]);
        #pragma unroll
        for (u32 c = 0; c < 4u; ++c) {
            const u32 lr = w + 8u * c, row = 32u * i + lr;
            if (row < T) {
                const float p0 = x0[c] / sum[c], p1 = x1[c] / sum[c];
                Ss[lr * SP + lane] = p0;
                if (wide) Ss[lr * SP + lane + 64u] = p1;
                if (lane < T) pout[row * T + lane] = p0;
                if (lane + 64u < T) pout[row * T + lane + 64u] = p1;
            }
        }
    }
    __syncthreads();
    if (w <= i) {                                           // the part of y_i that comes from the keys of tile w
        f16v acc; ZERO16(acc)
        tile_product(acc, Ss + 32u * w, SP, 1u, Vs + w * TILE, DP, 1u, r, h);
        put_partial(box, w, acc, lane);
    }
    __syncthreads();
    if (w < 4u) sum_and_store(y + (u64)b * T * y_pitch + (u64)hd * d, box, 0u, i + 1u, w, 32u * i, T, d, y_pitch, lane);
}
"""
        fmt = _fmt("P", "P", "P", "P", "P", "I", "I", "I", "I", "I", "I", "f")
    else:
        body = r"""
extern "C" __global__ __launch_bounds__(512) void attention_small_bwd(const float* __restrict__ q,
        const float* __restrict__ k, const float* __restrict__ v, const float* __restrict__ p, const float* __restrict__ y,
        const float* __restrict__ dy, float* __restrict__ dq, float* __restrict__ dk, float* __restrict__ dv,
        u32 T, u32 d, u32 pitch, u32 y_pitch, u32 g_pitch, u32 n_head, u32 nt, float scale) {
    __shared__ float Qs[4u * TILE], Ks[4u * TILE], Vs[4u * TILE], Gs[4u * TILE], dSs[4u * TILE], box[12u * 1024u], delta[128];
    const u32 bh = blockIdx.x / nt, i = blockIdx.x % nt, b = bh / n_head, hd = bh % n_head;
    const u32 t = threadIdx.x, w = t >> 6, lane = t & 63u, r = lane & 31u, h = lane >> 5;
    const u64 in_off = (u64)b * T * pitch + (u64)hd * d, y_off = (u64)b * T * y_pitch + (u64)hd * d;
    const u64 g_off = (u64)b * T * g_pitch + (u64)hd * d;
    const float* __restrict__ pin = p + (u64)bh * T * T;
    {   // q, dy (and delta) for rows from tile i on; k, v for rows up to tile i
        const u32 n_lo = 256u * (i + 1u), n_hi = 256u * (nt - i);
        float4 q4[2], g4[2], y4[2], k4[2], v4[2];
        #pragma unroll
        for (u32 n = 0; n < 2u; ++n) {
            const u32 it = t + 512u * n;
            if (it < n_hi) {
                q4[n] = head_part(q + in_off, it, 32u * i, T, d, pitch);
                g4[n] = head_part(dy + y_off, it, 32u * i, T, d, y_pitch);
                y4[n] = head_part(y + y_off, it, 32u * i, T, d, y_pitch);
            }
            if (it < n_lo) { k4[n] = head_part(k + in_off, it, 0u, T, d, pitch); v4[n] = head_part(v + in_off, it, 0u, T, d, pitch); }
        }
        #pragma unroll
        for (u32 n = 0; n < 2u; ++n) {
            const u32 it = t + 512u * n;
            if (it < n_hi) {
                put_part(Qs + i * TILE, it, q4[n]); put_part(Gs + i * TILE, it, g4[n]);
                float part = (g4[n].x * y4[n].x + g4[n].y * y4[n].y) + (g4[n].z * y4[n].z + g4[n].w * y4[n].w);
                part += dpp_f<DPP_XOR1>(part); part += dpp_f<DPP_XOR2>(part); part += dpp_f<DPP_HALF_MIRROR>(part);   // the row's 8 threads
                if ((it & 7u) == 0u) delta[32u * i + (it >> 3)] = part;
            }
            if (it < n_lo) { put_part(Ks, it, k4[n]); put_part(Vs, it, v4[n]); }
        }
    }
    __syncthreads();
    // wavefronts c and 4 + c share score tile (ti, tj): (i, c) for c <= i, (c, i) below it
    const u32 c = w & 3u, ti = c <= i ? i : c, tj = c <= i ? c : i;
    const bool live = ti < nt, column = tj == i;           // column: the tile feeds dk_i and dv_i (the diagonal tile does both)
    if (live && w < 4u) {
        float pe[16];                                       // the tile of P in accumulator layout, on its way while dP is computed
        #pragma unroll
        for (u32 e = 0; e < 16u; ++e) {
            const u32 row = 32u * ti + 8u * (e >> 2) + 4u * h + (e & 3u), col = 32u * tj + r;
            pe[e] = (row < T && col <= row) ? pin[row * T + col] : 0.0f;
        }
        f16v ds; ZERO16(ds)
        tile_product(ds, Gs + ti * TILE, DP, 1u, Vs + tj * TILE, 1u, DP, r, h);               // dP = dy_ti v_tj^T
        #pragma unroll
        for (u32 e = 0; e < 16u; ++e) {
            const u32 lr = 8u * (e >> 2) + 4u * h + (e & 3u);
            dSs[c * TILE + lr * DP + r] = (pe[e] * (ds[e] - delta[32u * ti + lr])) * scale;
        }
        wave_lds_fence();
        f16v acc; ZERO16(acc)
        if (ti == i) {                                      // dq_i, the part from the keys of tile tj
            tile_product(acc, dSs + c * TILE, DP, 1u, Ks + tj * TILE, DP, 1u, r, h);
            put_partial(box, tj, acc, lane);
        } else {                                            // dk_i, the part from the queries of tile ti
            tile_product(acc, dSs + c * TILE, 1u, DP, Qs + ti * TILE, DP, 1u, r, h);
            put_partial(box, 4u + ti, acc, lane);
        }
    }
    if (live && column && w >= 4u) {                        // dv_i, the part from the rows of tile ti: P(ti, i)^T dy_ti
        f16v acc; ZERO16(acc)
        float av[16], bv[16];
        #pragma unroll
        for (u32 s = 0; s < 16u; ++s) {
            const u32 row = 32u * ti + 2u * s + h, col = 32u * tj + r;
            av[s] = (row < T && col <= row) ? pin[row * T + col] : 0.0f;
            bv[s] = Gs[ti * TILE + (2u * s + h) * DP + r];
        }
        #pragma unroll
        for (u32 s = 0; s < 16u; ++s) acc = MFMA(av[s], bv[s], acc);
        put_partial(box, 8u + ti, acc, lane);
    }
    __syncthreads();
    if (w == 4u + i) {                                      // dk_i, the part from the diagonal tile, whose dS wavefront i wrote
        f16v acc; ZERO16(acc)
        tile_product(acc, dSs + i * TILE, 1u, DP, Qs + i * TILE, DP, 1u, r, h);
        put_partial(box, 4u + i, acc, lane);
    }
    __syncthreads();
    for (u32 job = w; job < 12u; job += 8u) {               // 3 outputs x 4 groups of accumulator entries
        const u32 out = job >> 2, g = job & 3u;
        if (out == 0u) sum_and_store(dq + g_off, box, 0u, i + 1u, g, 32u * i, T, d, g_pitch, lane);
        else if (out == 1u) sum_and_store(dk + g_off, box, 4u + i, 4u + nt, g, 32u * i, T, d, g_pitch, lane);
        else sum_and_store(dv + g_off, box, 8u + i, 8u + nt, g, 32u * i, T, d, g_pitch, lane);
    }
}
"""
        fmt = _fmt("P", "P", "P", "P", "P", "P", "P", "P", "P", "I", "I", "I", "I", "I", "I", "I", "f")
    return f"{PRELUDE}{WAVE_LDS_FENCE}{common}{body}", name, fmt


ATTN_FLASH_D = 64          # widest head the streaming attention kernels take (zero-padded to 32 or 64 columns in LDS)


@cache
def attention_flash_kernel(stage: str, DP: int, blocks_per_cu: int = 1) -> tuple[str, str, str]:
    """Causal self-attention for long sequences without the (T x T) probabilities in memory
    (examples/gpt.py:50-55 runs product, scale, mask, softmax, product and keeps four T x T tensors
    per head for the backward pass).  Heads of width d <= DP (DP = 32 or 64, d % 4 == 0) are read where
    they lie inside (B, T, pitch) tensors, zero-padded to DP columns on the chip.

    All products run on v_mfma_f32_32x32x2_f32 (lane l feeds A[l % 32][l / 32] and B[l / 32][l % 32]; entry e
    of a lane's accumulator is row 8 (e / 4) + 4 (l / 32) + e % 4, column l % 32).  The kernels are arranged so
    that the tile a wavefront has just computed is, entry for entry, the B operand of its next product: the
    sixteen rows a lane holds are exactly the k values it feeds in sixteen steps, in the order k = 8 (s / 4) +
    4 h + s % 4 for step s, and the A operand is read from LDS in the same order.  Nothing is transposed
    and no score passes through LDS.

      "fwd"    a block of four wavefronts per (sequence, head, 128 queries), a wavefront per 32 queries, which it
               holds in registers as the B operand of S^T = K Q^T.  The keys and values stream through LDS 64 at a
               time (double-buffered, the next tile in flight in registers).  In S^T a lane holds one query's
               scores against 32 of the 64 keys (the lane 32 further on holds the other 32), so the running
               maximum and sum of the online softmax are register operations and one exchange.  The
               probabilities exp(s * scale - m) feed O^T += V^T P^T; the accumulator is rescaled by
               exp(m_old - m_new) whenever a maximum moved and divided by the sum at the end.  The scores are kept in
               units of log2 (scale * log2 e is multiplied into the query registers once), so a probability is one
               subtraction and one hardware 2^x (1 ulp).  Besides the context
               y (B, T, y_pitch) the kernel writes lse = m + log(sum) per (sequence, head, query).
      "delta"  delta = rowsum(dy * y) per (sequence, head, query) (equal to rowsum(dP * P), since y = P v).
      "bwd"    a block per (sequence, head, 128 keys), a wavefront per 32 keys, whose key and value rows it holds
               in registers as B operands.  Queries stream through LDS 64 at a time with their dy rows, lse and
               delta: S = Q K^T again, P = exp(S * scale - lse), dP = dy V^T, dS = P (dP - delta) scale; then
               dV^T += dy^T P and dK^T += Q^T dS with P and dS as B operands straight from the accumulators.
               dS is written to ds (B, n_head, T, T) for the product dQ = dS K that follows (a plain
               lower-triangular product); query tiles above the diagonal inside the block's aligned group of
               256 are written as zeros, because that product reads whole tiles along the diagonal.
    Against the chain: 7 tile products per (query tile, key tile) pair instead of 6, and two passes over
    one T x T tensor per head instead of eleven over four; the sums are added in another order (2e-6 of the
    largest entry against float64)."""
    assert stage in ("fwd", "delta", "bwd") and DP in (32, 64) and blocks_per_cu in (1, 2)
    name = f"attention_flash_{stage}" + (f"_d{DP}" if stage != "delta" else "") + ("_o2" if blocks_per_cu == 2 else "")
    bounds = "256, 2" if blocks_per_cu == 2 else "256"           # "256, 2": registers held to what lets two blocks share a CU
    NB, ND, LP = DP // 8, DP // 32, DP + 4          # groups of 8 columns, 32-column tiles, LDS row pitch
    if stage == "delta":
        src = f"""{PRELUDE}
extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ dy, const float* __restrict__ y,
        float* __restrict__ delta, u32 rows, u32 T, u32 d, u32 y_pitch, u32 n_head) {{
    // sixteen lanes per (sequence, position, head): 16-byte items 0 .. 15 of the head's row
    const u32 item = blockIdx.x * 16u + (threadIdx.x >> 4), sub = threadIdx.x & 15u;
    float part = 0.0f;
    const bool live = item < rows;
    const u32 hd = live ? item % n_head : 0u, bt = live ? item / n_head : 0u;     // bt = b * T + t
    if (live && 4u * sub < d) {{
        const u64 at = (u64)bt * y_pitch + (u64)hd * d + 4u * sub;
        const float4 g = *reinterpret_cast<const float4*>(dy + at), o = *reinterpret_cast<const float4*>(y + at);
        part = (g.x * o.x + g.y * o.y) + (g.z * o.z + g.w * o.w);
    }}
    part += dpp_f<DPP_XOR1>(part);
    part += dpp_f<DPP_XOR2>(part);
    part += dpp_f<DPP_HALF_MIRROR>(part);
    part += dpp_f<DPP_MIRROR>(part);
    if (live && sub == 0u) delta[((u64)(bt / T) * n_head + hd) * T + bt % T] = part;
}}
"""
        return src, name, _fmt("P", "P", "P", "I", "I", "I", "I", "I")
    common = f"""
typedef float f16v __attribute__((ext_vector_type(16)));
#define DP {DP}u
#define NB {NB}u
#define ND {ND}u
#define LP {LP}u
#define MFMA(a, b, c) __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0)
#define ROW_OF(e, h) (8u * ((e) >> 2) + 4u * (h) + ((e) & 3u))
// 16-byte item `it` of rows [row0, ..) of a head: row row0 + it / (DP / 4), columns 4 (it % (DP / 4)) ..; zeros outside [0, T) x [0, d)
static __device__ __forceinline__ float4 head_item(const float* __restrict__ src, u32 it, u32 row0, u32 T, u32 d, u32 pitch) {{
    const u32 row = row0 + it / (DP / 4u), c4 = (it % (DP / 4u)) << 2;
    return (row < T && c4 < d) ? *reinterpret_cast<const float4*>(src + (u64)row * pitch + c4) : make_float4(0.f, 0.f, 0.f, 0.f);
}}
static __device__ __forceinline__ void put_item(float* __restrict__ tile, u32 it, const float4 v) {{
    *reinterpret_cast<float4*>(tile + (it / (DP / 4u)) * LP + ((it % (DP / 4u)) << 2)) = v;
}}
// the rows a lane holds as B operand: row `row` of a head, columns 8 blk + 4 h .. + 3 for blk = 0 .. NB - 1
static __device__ __forceinline__ void own_row(float4 (&reg)[{NB}], const float* __restrict__ src, u32 row, u32 h, u32 T, u32 d, u32 pitch) {{
    #pragma unroll
    for (u32 blk = 0; blk < NB; ++blk) {{
        const u32 c4 = 8u * blk + 4u * h;
        reg[blk] = (row < T && c4 < d) ? *reinterpret_cast<const float4*>(src + (u64)row * pitch + c4) : make_float4(0.f, 0.f, 0.f, 0.f);
    }}
}}
// acc += X Y^T for the 32 rows of X at `xs` (LDS, [row][LP]) and the 32 rows of Y that the lanes hold in `reg`
static __device__ __forceinline__ void rows_times_own(f16v& acc, const float* __restrict__ xs, const float4 (&reg)[{NB}], u32 r, u32 h) {{
    #pragma unroll
    for (u32 blk = 0; blk < NB; ++blk) {{
        const float4 a = *reinterpret_cast<const float4*>(xs + r * LP + 8u * blk + 4u * h);
        acc = MFMA(a.x, reg[blk].x, acc); acc = MFMA(a.y, reg[blk].y, acc);
        acc = MFMA(a.z, reg[blk].z, acc); acc = MFMA(a.w, reg[blk].w, acc);
    }}
}}
// acc (32 columns c0 .. of X^T, by the lanes' 32 columns) += X^T B, for the 32 rows of X at `xs` and B = the tile a lane holds in `b`
static __device__ __forceinline__ void cols_times_tile(f16v& acc, const float* __restrict__ xs, u32 c0, const f16v& b, u32 r, u32 h) {{
    #pragma unroll
    for (u32 st = 0; st < 16u; ++st) acc = MFMA(xs[ROW_OF(st, h) * LP + c0 + r], b[st], acc);
}}
"""
    if stage == "fwd":
        body = f"""
extern "C" __global__ __launch_bounds__({bounds}) void {name}(const float* __restrict__ q, const float* __restrict__ k,
        const float* __restrict__ v, float* __restrict__ y, float* __restrict__ lse,
        u32 T, u32 d, u32 pitch, u32 y_pitch, u32 n_head, u32 nq, float scale) {{
    __shared__ __attribute__((aligned(16))) float Ks[2][64u * LP], Vs[2][64u * LP];
    // the query tiles with the most keys first
    const u32 bh = blockIdx.x % (gridDim.x / nq), qi = nq - 1u - blockIdx.x / (gridDim.x / nq), b = bh / n_head, hd = bh % n_head;
    const u32 t = threadIdx.x, w = t >> 6, lane = t & 63u, r = lane & 31u, h = lane >> 5;
    const u64 in_off = (u64)b * T * pitch + (u64)hd * d;
    const u32 q0 = 128u * qi + 32u * w, query = q0 + r;                  // this wavefront's queries; this lane's
    const u32 n_kv = (min(T, 128u * qi + 128u) + 63u) / 64u;             // key tiles at or below the block's last query
    float4 qreg[{NB}];
    own_row(qreg, q + in_off, query, h, T, d, pitch);
    const float s2 = scale * 1.44269504088896340736f;                    // scores are kept in units of log2: exp(x) = 2^(x log2 e)
    #pragma unroll
    for (u32 blk = 0; blk < NB; ++blk) {{ qreg[blk].x *= s2; qreg[blk].y *= s2; qreg[blk].z *= s2; qreg[blk].w *= s2; }}
    f16v o[{ND}];
    #pragma unroll
    for (u32 dt = 0; dt < ND; ++dt) {{ _Pragma("unroll") for (int z = 0; z < 16; ++z) o[dt][z] = 0.0f; }}
    float m_run = -__builtin_inff(), l_run = 0.0f;
    constexpr u32 NI = 64u * (DP / 4u) / 256u;                           // 16-byte items per thread and tile
    float4 kn[NI], vn[NI];
    auto fetch = [&](u32 j) {{
        #pragma unroll
        for (u32 n = 0; n < NI; ++n) {{
            kn[n] = head_item(k + in_off, t + 256u * n, 64u * j, T, d, pitch);
            vn[n] = head_item(v + in_off, t + 256u * n, 64u * j, T, d, pitch);
        }}
    }};
    auto stash = [&](u32 buf) {{
        #pragma unroll
        for (u32 n = 0; n < NI; ++n) {{ put_item(Ks[buf], t + 256u * n, kn[n]); put_item(Vs[buf], t + 256u * n, vn[n]); }}
    }};
    fetch(0u);
    stash(0u);
    __syncthreads();
    for (u32 j = 0; j < n_kv; ++j) {{
        const u32 buf = j & 1u, kv0 = 64u * j;
        if (j + 1u < n_kv) fetch(j + 1u);
        if (kv0 <= q0 + 31u) {{                                          // some key of the tile is visible to some query of the wavefront
            f16v s[2];
            #pragma unroll
            for (u32 kt = 0; kt < 2u; ++kt) {{
                _Pragma("unroll") for (int z = 0; z < 16; ++z) s[kt][z] = 0.0f;
                rows_times_own(s[kt], Ks[buf] + 32u * kt * LP, qreg, r, h);          // S^T: keys by queries
            }}
            if (kv0 + 63u > q0) {{                                       // some key of the tile lies beyond some query: the causal mask
                #pragma unroll
                for (u32 kt = 0; kt < 2u; ++kt)
                    #pragma unroll
                    for (u32 e = 0; e < 16u; ++e) if (kv0 + 32u * kt + ROW_OF(e, h) > query) s[kt][e] = -__builtin_inff();
            }}
            float mx = -__builtin_inff();
            #pragma unroll
            for (u32 kt = 0; kt < 2u; ++kt)
                #pragma unroll
                for (u32 e = 0; e < 16u; ++e) mx = fmaxf(mx, s[kt][e]);
            mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
            const float m_new = fmaxf(m_run, mx);                        // finite: key 0 is visible to every query
            float part = 0.0f;
            #pragma unroll
            for (u32 kt = 0; kt < 2u; ++kt)
                #pragma unroll
                for (u32 e = 0; e < 16u; ++e) {{ const float pe = __builtin_amdgcn_exp2f(s[kt][e] - m_new); s[kt][e] = pe; part += pe; }}
            if (__any(m_new != m_run)) {{                                // (a maximum that stays is the rule after the first few tiles)
                const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
                l_run *= alpha;
                #pragma unroll
                for (u32 dt = 0; dt < ND; ++dt) {{ _Pragma("unroll") for (int z = 0; z < 16; ++z) o[dt][z] *= alpha; }}
                m_run = m_new;
            }}
            l_run += part;
            #pragma unroll
            for (u32 dt = 0; dt < ND; ++dt)
                #pragma unroll
                for (u32 kt = 0; kt < 2u; ++kt) cols_times_tile(o[dt], Vs[buf] + 32u * kt * LP, 32u * dt, s[kt], r, h);    // O^T += V^T P^T
        }}
        if (j + 1u < n_kv) stash(buf ^ 1u);
        __syncthreads();
    }}
    const float l = l_run + __shfl_xor(l_run, 32, WAVE);
    if (query < T) {{
        if (h == 0u) lse[(u64)bh * T + query] = (m_run + log2f(l)) * 0.69314718055994530942f;
        float* __restrict__ yrow = y + (u64)b * T * y_pitch + (u64)query * y_pitch + (u64)hd * d;
        #pragma unroll
        for (u32 dt = 0; dt < ND; ++dt)
            #pragma unroll
            for (u32 g = 0; g < 4u; ++g) {{
                const u32 col = 32u * dt + 8u * g + 4u * h;
                if (col < d) *reinterpret_cast<float4*>(yrow + col) =
                    make_float4(o[dt][4u * g] / l, o[dt][4u * g + 1u] / l, o[dt][4u * g + 2u] / l, o[dt][4u * g + 3u] / l);
            }}
    }}
}}
"""
        fmt = _fmt("P", "P", "P", "P", "P", "I", "I", "I", "I", "I", "I", "f")
    else:
        body = f"""
extern "C" __global__ __launch_bounds__({bounds}) void {name}(const float* __restrict__ q, const float* __restrict__ k,
        const float* __restrict__ v, const float* __restrict__ dy, const float* __restrict__ lse, const float* __restrict__ delta,
        float* __restrict__ ds, float* __restrict__ dk, float* __restrict__ dv,
        u32 T, u32 d, u32 pitch, u32 y_pitch, u32 g_pitch, u32 n_head, u32 nk, float scale) {{
    __shared__ __attribute__((aligned(16))) float Qs[2][64u * LP], Gs[2][64u * LP], Ls[2][64], Ds[2][64];
    // the key tiles with the most queries first
    const u32 bh = blockIdx.x % (gridDim.x / nk), ki = blockIdx.x / (gridDim.x / nk), b = bh / n_head, hd = bh % n_head;
    const u32 t = threadIdx.x, w = t >> 6, lane = t & 63u, r = lane & 31u, h = lane >> 5;
    const u64 in_off = (u64)b * T * pitch + (u64)hd * d, y_off = (u64)b * T * y_pitch + (u64)hd * d;
    const u32 k0 = 128u * ki + 32u * w, key = k0 + r;                    // this wavefront's keys; this lane's
    const u32 j0 = (128u * ki / 256u) * 4u, nq = (T + 63u) / 64u;         // query tiles from the start of the aligned group of 256
    float4 kreg[{NB}], vreg[{NB}];
    own_row(kreg, k + in_off, key, h, T, d, pitch);
    own_row(vreg, v + in_off, key, h, T, d, pitch);
    const float s2 = scale * 1.44269504088896340736f;                    // scores in units of log2, as in the forward pass
    #pragma unroll
    for (u32 blk = 0; blk < NB; ++blk) {{ kreg[blk].x *= s2; kreg[blk].y *= s2; kreg[blk].z *= s2; kreg[blk].w *= s2; }}
    f16v gk[{ND}], gv[{ND}];
    #pragma unroll
    for (u32 dt = 0; dt < ND; ++dt) {{ _Pragma("unroll") for (int z = 0; z < 16; ++z) {{ gk[dt][z] = 0.0f; gv[dt][z] = 0.0f; }} }}
    constexpr u32 NI = 64u * (DP / 4u) / 256u;
    float4 qn[NI], gn[NI];
    float ln = 0.0f, dn = 0.0f;
    const float* __restrict__ lrow = lse + (u64)bh * T;
    const float* __restrict__ drow = delta + (u64)bh * T;
    float* __restrict__ dsout = ds + (u64)bh * T * T;
    auto fetch = [&](u32 j) {{
        #pragma unroll
        for (u32 n = 0; n < NI; ++n) {{
            qn[n] = head_item(q + in_off, t + 256u * n, 64u * j, T, d, pitch);
            gn[n] = head_item(dy + y_off, t + 256u * n, 64u * j, T, d, y_pitch);
        }}
        if (t < 64u) {{ const u32 row = 64u * j + t; ln = row < T ? lrow[row] * 1.44269504088896340736f : __builtin_inff(); dn = row < T ? drow[row] : 0.0f; }}
    }};
    auto stash = [&](u32 buf) {{
        #pragma unroll
        for (u32 n = 0; n < NI; ++n) {{ put_item(Qs[buf], t + 256u * n, qn[n]); put_item(Gs[buf], t + 256u * n, gn[n]); }}
        if (t < 64u) {{ Ls[buf][t] = ln; Ds[buf][t] = dn; }}
    }};
    fetch(j0);
    stash(0u);
    __syncthreads();
    for (u32 j = j0; j < nq; ++j) {{
        const u32 buf = (j - j0) & 1u, qt0 = 64u * j;
        if (j + 1u < nq) fetch(j + 1u);
        #pragma unroll
        for (u32 qt = 0; qt < 2u; ++qt) {{
            const u32 row0 = qt0 + 32u * qt;                             // first query of this 32 x 32 tile
            f16v p, dsv;
            _Pragma("unroll") for (int z = 0; z < 16; ++z) {{ p[z] = 0.0f; dsv[z] = 0.0f; }}
            const bool live = row0 + 31u >= k0;                           // some query of the tile sees some key of the wavefront
            if (live) {{
                rows_times_own(p, Qs[buf] + 32u * qt * LP, kreg, r, h);              // S: queries by keys
                rows_times_own(dsv, Gs[buf] + 32u * qt * LP, vreg, r, h);            // dP = dy V^T
                #pragma unroll
                for (u32 e = 0; e < 16u; ++e) {{
                    const u32 lr = 32u * qt + ROW_OF(e, h);
                    const float pe = __builtin_amdgcn_exp2f(p[e] - Ls[buf][lr]);                        // (rows beyond T: lse = +inf)
                    p[e] = pe;
                    dsv[e] = (pe * (dsv[e] - Ds[buf][lr])) * scale;
                }}
                if (k0 + 31u > row0) {{                                   // the tile straddles the diagonal: nothing above it
                    #pragma unroll
                    for (u32 e = 0; e < 16u; ++e) if (key > row0 + ROW_OF(e, h)) {{ p[e] = 0.0f; dsv[e] = 0.0f; }}
                }}
                #pragma unroll
                for (u32 dt = 0; dt < ND; ++dt) {{
                    cols_times_tile(gv[dt], Gs[buf] + 32u * qt * LP, 32u * dt, p, r, h);       // dV^T += dy^T P
                    cols_times_tile(gk[dt], Qs[buf] + 32u * qt * LP, 32u * dt, dsv, r, h);     // dK^T += Q^T dS
                }}
            }}
            if (key < T) {{
                #pragma unroll
                for (u32 e = 0; e < 16u; ++e) {{
                    const u32 row = row0 + ROW_OF(e, h);
                    if (row < T) dsout[(u64)row * T + key] = dsv[e];
                }}
            }}
        }}
        if (j + 1u < nq) stash(buf ^ 1u);
        __syncthreads();
    }}
    if (key < T) {{
        const u64 g_off = (u64)b * T * g_pitch + (u64)key * g_pitch + (u64)hd * d;
        #pragma unroll
        for (u32 dt = 0; dt < ND; ++dt)
            #pragma unroll
            for (u32 g = 0; g < 4u; ++g) {{
                const u32 col = 32u * dt + 8u * g + 4u * h;
                if (col < d) {{
                    *reinterpret_cast<float4*>(dk + g_off + col) = make_float4(gk[dt][4u * g], gk[dt][4u * g + 1u], gk[dt][4u * g + 2u], gk[dt][4u * g + 3u]);
                    *reinterpret_cast<float4*>(dv + g_off + col) = make_float4(gv[dt][4u * g], gv[dt][4u * g + 1u], gv[dt][4u * g + 2u], gv[dt][4u * g + 3u]);
                }}
            }}
    }}
}}
"""
        fmt = _fmt("P", "P", "P", "P", "P", "P", "P", "P", "P", "I", "I", "I", "I", "I", "I", "I", "f")
    return f"{PRELUDE}{common}{body}", name, fmt


@cache
def adam_multi_inplace_kernel() -> tuple[str, str, str]:
    """adam_inplace_kernel for a whole parameter list in one launch.  `ptrs` holds four rows of
    addresses (p, g, m, v) per tensor, `sizes` the element counts, `first` the first block of each
    tensor and `owner` the tensor of every block; a block updates 1024 consecutive elements of its
    tensor (16-byte accesses: every address is 16-byte aligned, the n % 4 tail is done by the
    tensor's first block) -- or 64 of them when the gradient is a pending sum of more than 16 parts,
    whose addition the block's threads then share.  Same arithmetic as the per-tensor kernel, so the same bits.

    `rows_of` holds two numbers per tensor: how many parts its gradient pointer holds and how many floats
    lie between one part and the next.  1 part: the gradient itself.  More: parts whose sum is the
    gradient (the batch entries of a weight gradient -- for a third of a stacked weight one whole stacked
    gradient apart -- or the partial rows of an RMSNorm gain).  They are added up here, element by element, in
    exactly the order reduce_cols_kernel adds a column of that many rows (thread rows 4 or 16 apart,
    four running sums each, joined pairwise, then the thread rows in order), so the update has the bits
    it would have had with the column-sum launch in between."""
    src, _, _ = adam_kernel(4)
    head = src[:src.index('extern "C"')]
    name = "adam_multi_inplace"
    colsum = r"""
// Sum over l of row l of a (rows, n) array at one place -- element j, or the four elements of 16-byte item j when
// n is a multiple of 4 -- in reduce_cols_kernel's order.
static __device__ __forceinline__ float ld_at(const float* __restrict__ g, u64 row_off, u32 j, float) { return g[row_off + j]; }
static __device__ __forceinline__ float4 ld_at(const float* __restrict__ g, u64 row_off, u32 j, float4) {
    return reinterpret_cast<const float4*>(g + row_off)[j];
}
static __device__ __forceinline__ float add2(float a, float b) { return a + b; }
static __device__ __forceinline__ float4 add2(float4 a, float4 b) { return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w); }
static __device__ __forceinline__ void zero_of(float& z) { z = 0.0f; }
static __device__ __forceinline__ void zero_of(float4& z) { z = make_float4(0.f, 0.f, 0.f, 0.f); }
template <int TY, typename T> static __device__ __forceinline__ T colsum(const float* __restrict__ g, u32 rows, u32 n, u32 j) {
    T r; zero_of(r);
    #pragma unroll 1
    for (u32 ty = 0; ty < (u32)TY; ++ty) {
        T a0, a1, a2, a3; zero_of(a0); zero_of(a1); zero_of(a2); zero_of(a3);
        u32 l = ty;
        for (; l + 3u * TY < rows; l += 4u * TY) {
            const T t0 = ld_at(g, (u64)l * n, j, T()), t1 = ld_at(g, (u64)(l + TY) * n, j, T());
            const T t2 = ld_at(g, (u64)(l + 2u * TY) * n, j, T()), t3 = ld_at(g, (u64)(l + 3u * TY) * n, j, T());
            a0 = add2(a0, t0); a1 = add2(a1, t1); a2 = add2(a2, t2); a3 = add2(a3, t3);
        }
        for (; l < rows; l += TY) a0 = add2(a0, ld_at(g, (u64)l * n, j, T()));
        a0 = add2(a0, a1); a2 = add2(a2, a3); a0 = add2(a0, a2);
        r = ty == 0u ? a0 : add2(r, a0);
    }
    return r;
}
// colsum<4> for up to 16 rows (the batch entries of a weight gradient, the partial rows of a gain): the same additions
// in the same order, with every row's load issued before the first of them instead of four rounds of four
template <typename T> static __device__ __forceinline__ T colsum16(const float* __restrict__ g, u32 rows, u32 n, u32 j) {
    T t[16];
    #pragma unroll
    for (u32 l = 0; l < 16u; ++l) { zero_of(t[l]); if (l < rows) t[l] = ld_at(g, (u64)l * n, j, T()); }
    T r; zero_of(r);
    #pragma unroll
    for (u32 ty = 0; ty < 4u; ++ty) {
        T a0, a1, a2, a3; zero_of(a0); zero_of(a1); zero_of(a2); zero_of(a3);
        if (ty + 12u < rows) { a0 = add2(a0, t[ty]); a1 = add2(a1, t[ty + 4u]); a2 = add2(a2, t[ty + 8u]); a3 = add2(a3, t[ty + 12u]); }
        else {
            #pragma unroll
            for (u32 l = ty; l < 16u; l += 4u) if (l < rows) a0 = add2(a0, t[l]);
        }
        a0 = add2(a0, a1); a2 = add2(a2, a3); a0 = add2(a0, a2);
        r = ty == 0u ? a0 : add2(r, a0);
    }
    return r;
}
// n: floats from one row to the next
template <typename T> static __device__ __forceinline__ T grad_at(const float* __restrict__ g, u32 rows, u32 n, u32 j) {
    if (rows == 1u) return ld_at(g, 0, j, T());
    if (rows <= 16u) return colsum16<T>(g, rows, n, j);
    return rows > 64u ? colsum<16, T>(g, rows, n, j) : colsum<4, T>(g, rows, n, j);
}
"""
    src2 = f"""{head}{colsum}extern "C" __global__ __launch_bounds__(256) void {name}(const u64* __restrict__ ptrs,
        const u32* __restrict__ sizes, const u32* __restrict__ first, const u32* __restrict__ owner,
        const u32* __restrict__ rows_of, u32 n_tensors, const AdamArgs* __restrict__ ap) {{
    const AdamArgs a = *ap;
    const u32 t = owner[blockIdx.x];
    const u32 lb = blockIdx.x - first[t];
    float* p = reinterpret_cast<float*>(ptrs[t]);
    const float* __restrict__ g = reinterpret_cast<const float*>(ptrs[n_tensors + t]);
    float* m = reinterpret_cast<float*>(ptrs[2u * n_tensors + t]);
    float* v = reinterpret_cast<float*>(ptrs[3u * n_tensors + t]);
    const u32 n = sizes[t], nv = n >> 2, rows = rows_of[2u * t], gp = rows_of[2u * t + 1u];       // parts of the gradient and their distance
    if (rows > 16u && (n & 3u) == 0u) {{
        // Many parts (the per-wavefront partial rows of an RMSNorm gain): a block takes 16 columns of 16 bytes and adds
        // them up the way a 64 x 16 block of the column-sum kernel does -- thread row ty owns parts ty, ty + TY, ..
        // in four running sums, joined pairwise; then the thread rows are added in order.
        __shared__ float4 part[16][16];
        const u32 ty = threadIdx.x >> 4, cx = threadIdx.x & 15u, col = lb * 16u + cx;
        const u32 TY = rows > 64u ? 16u : 4u;
        if (col < nv && ty < TY) {{
            float4 a0, a1, a2, a3; zero_of(a0); zero_of(a1); zero_of(a2); zero_of(a3);
            u32 l = ty;
            for (; l + 3u * TY < rows; l += 4u * TY) {{
                const float4 t0 = ld_at(g, (u64)l * gp, col, float4()), t1 = ld_at(g, (u64)(l + TY) * gp, col, float4());
                const float4 t2 = ld_at(g, (u64)(l + 2u * TY) * gp, col, float4()), t3 = ld_at(g, (u64)(l + 3u * TY) * gp, col, float4());
                a0 = add2(a0, t0); a1 = add2(a1, t1); a2 = add2(a2, t2); a3 = add2(a3, t3);
            }}
            for (; l < rows; l += TY) a0 = add2(a0, ld_at(g, (u64)l * gp, col, float4()));
            a0 = add2(a0, a1); a2 = add2(a2, a3); a0 = add2(a0, a2);
            part[ty][cx] = a0;
        }}
        __syncthreads();
        if (ty == 0u && col < nv) {{
            float4 g4 = part[0][cx];
            for (u32 k = 1; k < TY; ++k) g4 = add2(g4, part[k][cx]);
            const float4 p4 = reinterpret_cast<float4*>(p)[col];
            const float4 m4 = reinterpret_cast<float4*>(m)[col], v4 = reinterpret_cast<float4*>(v)[col];
            float4 po, mo, vo;
            adam1(p4.x, g4.x, m4.x, v4.x, a, po.x, mo.x, vo.x);
            adam1(p4.y, g4.y, m4.y, v4.y, a, po.y, mo.y, vo.y);
            adam1(p4.z, g4.z, m4.z, v4.z, a, po.z, mo.z, vo.z);
            adam1(p4.w, g4.w, m4.w, v4.w, a, po.w, mo.w, vo.w);
            reinterpret_cast<float4*>(p)[col] = po;
            reinterpret_cast<float4*>(m)[col] = mo;
            reinterpret_cast<float4*>(v)[col] = vo;
        }}
        return;
    }}
    const u32 i = lb * 256u + threadIdx.x;
    if (i < nv) {{
        float4 g4;
        if ((n & 3u) == 0u) g4 = grad_at<float4>(g, rows, gp, i);         // every part starts 16-byte aligned
        else {{ g4.x = grad_at<float>(g, rows, gp, 4u * i); g4.y = grad_at<float>(g, rows, gp, 4u * i + 1u);
               g4.z = grad_at<float>(g, rows, gp, 4u * i + 2u); g4.w = grad_at<float>(g, rows, gp, 4u * i + 3u); }}
        const float4 p4 = reinterpret_cast<float4*>(p)[i];
        const float4 m4 = reinterpret_cast<float4*>(m)[i], v4 = reinterpret_cast<float4*>(v)[i];
        float4 po, mo, vo;
        adam1(p4.x, g4.x, m4.x, v4.x, a, po.x, mo.x, vo.x);
        adam1(p4.y, g4.y, m4.y, v4.y, a, po.y, mo.y, vo.y);
        adam1(p4.z, g4.z, m4.z, v4.z, a, po.z, mo.z, vo.z);
        adam1(p4.w, g4.w, m4.w, v4.w, a, po.w, mo.w, vo.w);
        reinterpret_cast<float4*>(p)[i] = po;
        reinterpret_cast<float4*>(m)[i] = mo;
        reinterpret_cast<float4*>(v)[i] = vo;
    }}
    if (lb == 0 && threadIdx.x < (n & 3u)) {{
        const u32 j = (nv << 2) + threadIdx.x;
        float po, mo, vo;
        adam1(p[j], grad_at<float>(g, rows, gp, j), m[j], v[j], a, po, mo, vo);
        p[j] = po; m[j] = mo; v[j] = vo;
    }}
}}
"""
    return src2, name, _fmt("P", "P", "P", "P", "P", "I", "P")


@cache
def sgd_inplace_kernel(momentum: bool) -> tuple[str, str, str]:
    """p -= (momentum ? (v = v * mu + g) : g) * lr, in place (dlgrad/nn/optim.py:22-45): the
    form a captured graph can replay, since no buffer changes its address.  fp contraction is
    off, so the two or four roundings are those of the op-by-op expression."""
    name = f"sgd_step_inplace{'_mom' if momentum else ''}"
    src = f"""{PRELUDE}
extern "C" __global__ __launch_bounds__(256) void {name}(float* p, const float* __restrict__ g, float* v,
        u32 n, float lr, float mu) {{
    #pragma clang fp contract(off)
    const u32 j = blockIdx.x * 256u + threadIdx.x;
    if (j < n) {{
        float upd = g[j];
        {'{ const float t = v[j] * mu; upd = t + upd; v[j] = upd; }' if momentum else '(void)v; (void)mu;'}
        const float t2 = upd * lr;
        p[j] = p[j] - t2;
    }}
}}
"""
    return src, name, _fmt("P", "P", "P", "I", "f", "f")


SGD_MULTI_MAX = 16


@cache
def sgd_multi_inplace_kernel(momentum: bool) -> tuple[str, str, str]:
    """sgd_inplace_kernel for up to SGD_MULTI_MAX parameters in one launch.  Their addresses and sizes travel
    in the kernel's argument block, so nothing is uploaded and a captured step replays with them; block b
    works on the parameter whose first block is the last one not after b (unused entries hold the total).
    Same statements, same roundings as the launch per parameter."""
    name = f"sgd_multi_inplace{'_mom' if momentum else ''}"
    M = SGD_MULTI_MAX
    src = f"""{PRELUDE}
struct SgdArgs {{ float* p[{M}]; const float* g[{M}]; float* v[{M}]; u32 first[{M}]; u32 n[{M}]; float lr, mu; }};
extern "C" __global__ __launch_bounds__(256) void {name}(SgdArgs a) {{
    #pragma clang fp contract(off)
    float* p = a.p[0]; const float* g = a.g[0]; float* v = a.v[0];
    u32 first = 0u, n = a.n[0];
    #pragma unroll
    for (u32 k = 1; k < {M}u; ++k)
        if (blockIdx.x >= a.first[k]) {{ p = a.p[k]; g = a.g[k]; v = a.v[k]; first = a.first[k]; n = a.n[k]; }}
    const u32 j = (blockIdx.x - first) * 256u + threadIdx.x;
    if (j < n) {{
        float upd = g[j];
        {'{ const float t = v[j] * a.mu; upd = t + upd; v[j] = upd; }' if momentum else '(void)v;'}
        const float t2 = upd * a.lr;
        p[j] = p[j] - t2;
    }}
}}
"""
    return src, name, "@" + "P" * (3 * M) + "I" * (2 * M) + "ff"


@cache
def adam_inplace_kernel(vec: int) -> tuple[str, str, str]:
    """adam_kernel's arithmetic applied in place to p, m and v, with the eight constants read
    from device memory.  This is the form a captured graph can replay: the addresses never
    change and the step-dependent bias corrections are refreshed by a small upload before
    each replay instead of being frozen into the kernel arguments."""
    src, name, _ = adam_kernel(vec)
    name2 = f"adam_step_inplace_v{vec}"
    i = src.index('extern "C"')
    head = src[:i]
    if vec == 4:
        body = """
    const AdamArgs a = *ap;
    const u32 nv = n >> 2;
    const u32 i = blockIdx.x * 256u + threadIdx.x;
    if (i < nv) {
        const float4 p4 = reinterpret_cast<float4*>(p)[i], g4 = reinterpret_cast<const float4*>(g)[i];
        const float4 m4 = reinterpret_cast<float4*>(m)[i], v4 = reinterpret_cast<float4*>(v)[i];
        float4 po, mo, vo;
        adam1(p4.x, g4.x, m4.x, v4.x, a, po.x, mo.x, vo.x);
        adam1(p4.y, g4.y, m4.y, v4.y, a, po.y, mo.y, vo.y);
        adam1(p4.z, g4.z, m4.z, v4.z, a, po.z, mo.z, vo.z);
        adam1(p4.w, g4.w, m4.w, v4.w, a, po.w, mo.w, vo.w);
        reinterpret_cast<float4*>(p)[i] = po;
        reinterpret_cast<float4*>(m)[i] = mo;
        reinterpret_cast<float4*>(v)[i] = vo;
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3u)) {
        const u32 j = (nv << 2) + threadIdx.x;
        float po, mo, vo;
        adam1(p[j], g[j], m[j], v[j], a, po, mo, vo);
        p[j] = po; m[j] = mo; v[j] = vo;
    }
"""
    else:
        body = """
    const AdamArgs a = *ap;
    const u32 j = blockIdx.x * 256u + threadIdx.x;
    if (j < n) { float po, mo, vo; adam1(p[j], g[j], m[j], v[j], a, po, mo, vo); p[j] = po; m[j] = mo; v[j] = vo; }
"""
    src2 = f"""{head}extern "C" __global__ __launch_bounds__(256) void {name2}(float* p, const float* __restrict__ g,
        float* m, float* v, u32 n, const AdamArgs* __restrict__ ap) {{
{body}}}
"""
    return src2, name2, _fmt("P", "P", "P", "P", "I", "P")


@cache
def adam_kernel(vec: int) -> tuple[str, str, str]:
    """One Adam update of one parameter tensor: the fourteen element-wise kernels of
    dlgrad/nn/optim.py:59-70 in a single pass, writing new p, m and v buffers.

    Every operation is the same fp32 operation, in the same order, as in the unfused
    expression, and fp contraction is switched off so that no a*b+c becomes an fma: the
    result is bit-identical to the op-by-op path:
        m' = m*b1 + g*(1-b1);  v' = v*b2 + (g*g)*(1-b2)
        p' = p - ((m'/c1) / (sqrt(v'/c2) + eps)) * lr        (c1 = 1-b1^t, c2 = 1-b2^t)"""
    name = f"adam_step_v{vec}"
    step = """
static __device__ __forceinline__ void adam1(float p, float g, float m, float v, const AdamArgs& a,
                                             float& po, float& mo, float& vo) {
    #pragma clang fp contract(off)
    const float t1 = m * a.b1, t2 = g * a.omb1;
    mo = t1 + t2;
    const float gg = g * g;
    const float t3 = v * a.b2, t4 = gg * a.omb2;
    vo = t3 + t4;
    const float mh = mo / a.c1, vh = vo / a.c2;
    const float den = sqrtf(vh) + a.eps;
    const float q = mh / den;
    po = p - q * a.lr;
}
"""
    if vec == 4:
        body = """
    const u32 nv = n >> 2;
    const u32 i = blockIdx.x * 256u + threadIdx.x;
    if (i < nv) {
        const float4 p4 = reinterpret_cast<const float4*>(p)[i], g4 = reinterpret_cast<const float4*>(g)[i];
        const float4 m4 = reinterpret_cast<const float4*>(m)[i], v4 = reinterpret_cast<const float4*>(v)[i];
        float4 po, mo, vo;
        adam1(p4.x, g4.x, m4.x, v4.x, a, po.x, mo.x, vo.x);
        adam1(p4.y, g4.y, m4.y, v4.y, a, po.y, mo.y, vo.y);
        adam1(p4.z, g4.z, m4.z, v4.z, a, po.z, mo.z, vo.z);
        adam1(p4.w, g4.w, m4.w, v4.w, a, po.w, mo.w, vo.w);
        reinterpret_cast<float4*>(p_out)[i] = po;
        reinterpret_cast<float4*>(m_out)[i] = mo;
        reinterpret_cast<float4*>(v_out)[i] = vo;
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3u)) {
        const u32 j = (nv << 2) + threadIdx.x;
        adam1(p[j], g[j], m[j], v[j], a, p_out[j], m_out[j], v_out[j]);
    }
"""
    else:
        body = """
    const u32 j = blockIdx.x * 256u + threadIdx.x;
    if (j < n) adam1(p[j], g[j], m[j], v[j], a, p_out[j], m_out[j], v_out[j]);
"""
    src = f"""{PRELUDE}
struct AdamArgs {{ float b1, omb1, b2, omb2, c1, c2, eps, lr; }};
{step}
extern "C" __global__ __launch_bounds__(256) void {name}(const float* __restrict__ p,
        const float* __restrict__ g, const float* __restrict__ m, const float* __restrict__ v,
        float* __restrict__ p_out, float* __restrict__ m_out, float* __restrict__ v_out, u32 n, AdamArgs a) {{
{body}}}
"""
    return src, name, _fmt("P", "P", "P", "P", "P", "P", "P", "I", "8f")
