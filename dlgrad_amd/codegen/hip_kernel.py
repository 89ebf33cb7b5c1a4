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
    fargs = ", ".join([f"float x{k}" for k in range(nx)] + [f"float s{k}" for k in range(n_sval_extra)] + ["u32 i"])
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
                loads += f"            r{k}[u] = reinterpret_cast<const float4*>(a{k})[v];\n"
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
            calc += f"            o.{c} = f({xs}{extra}(v << 2) + {j});\n"
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
        out[i] = f({tail_x}{extra}i);
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
        if (i < n) out[i] = f({xs}{extra}i);
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
