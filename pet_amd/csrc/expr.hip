// Memory-bound operators given as an index expression (MemBoundOp,
// src/Graph/operator.cc:3601-3644): every output element is the value of a small
// expression over the output position: reads of input tensors at computed indices (zero
// outside the tensor), sums over iterators, arithmetic, ReLU / tanh. The reference evaluates
// the expression tree on the host (nnet::Interpreter, src/nnet/Visitor/Interpreter.cc) and
// prints a TVM kernel for the GPU (src/Graph/code_engine.cc:1752-1798); here the tree is
// flattened by the caller into the integer program described in pet_hip.h and one thread per
// output element runs it. Control flow depends on the program only, except a padded range
// that answers 0, so the lanes of a wave stay together almost everywhere.
#include "common.h"

using namespace pet;

namespace {

constexpr int kMaxTensors = 8;
constexpr int kMaxVars = 32;
constexpr int kStack = 16;
constexpr int kMaxLdsCode = 4096; // program words kept in LDS

struct ExprParams {
    const int *code; // device copy of the program
    int ncode;
    int pc0;         // first instruction
    const float *in[kMaxTensors];
    int nd[kMaxTensors];
    int shape_at[kMaxTensors]; // index into code of each tensor's shape
    float *out;
    unsigned total;
    int out_nd;
    int out_shape[PET_HIP_MAX_RANK];
};

// Interpreter state lives in LDS, one column per thread ([slot][thread]: a wave's accesses
// to one slot are consecutive banks); arrays indexed at run time would otherwise sit in
// scratch memory, a round trip through the cache per push and pop. The program is copied to
// LDS too when it fits (kMaxLdsCode words), so an instruction fetch is an LDS broadcast.
template <bool CODE_IN_LDS>
__global__ __launch_bounds__(256) void expr_kernel(ExprParams p) {
    extern __shared__ __attribute__((aligned(16))) int smem[];
    const int nt = blockDim.x, tid = threadIdx.x;
    int *istack = smem + tid;                    // slot s at istack[s * nt]
    int *fbits = smem + kStack * nt + tid;       // value stack, as bit patterns
    int *vars = smem + 2 * kStack * nt + tid;
    int *tab = smem + (2 * kStack + kMaxVars) * nt; // [nd x 8][shape_at x 8]
    int *lcode = tab + 2 * kMaxTensors;
    if (tid < kMaxTensors) {
        tab[tid] = p.nd[tid];
        tab[kMaxTensors + tid] = p.shape_at[tid];
    }
    if (CODE_IN_LDS)
        for (int j = tid; j < p.ncode; j += nt)
            lcode[j] = p.code[j];
    __syncthreads();
    const unsigned i = blockIdx.x * (unsigned)nt + tid;
    if (i >= p.total)
        return;
    const int *__restrict__ c = CODE_IN_LDS ? lcode : p.code;
#define IS(s) istack[(s) * nt]
#define FS(s) (*reinterpret_cast<float *>(&fbits[(s) * nt]))
#define VAR(s) vars[(s) * nt]
    int isp = 0, fsp = 0;
    // the output position, outermost dim first, is what the outermost range pops
    {
        unsigned t = i;
        for (int j = p.out_nd - 1; j >= 0; --j) {
            const unsigned e = (unsigned)c[p.pc0 - p.out_nd + j];
            IS(j) = (int)(t % e);
            t /= e;
        }
        isp = p.out_nd;
    }
    int pc = p.pc0;
    for (;;) {
        const int op = c[pc];
        if (op == PET_HIP_EXPR_END)
            break;
        switch (op) {
        case PET_HIP_EXPR_ICONST:
            IS(isp) = c[pc + 1];
            ++isp;
            pc += 2;
            break;
        case PET_HIP_EXPR_IVAR:
            IS(isp) = VAR(c[pc + 1]);
            ++isp;
            pc += 2;
            break;
        case PET_HIP_EXPR_IADD:
        case PET_HIP_EXPR_ISUB:
        case PET_HIP_EXPR_IMUL:
        case PET_HIP_EXPR_IDIV:
        case PET_HIP_EXPR_IMOD: {
            const int b = IS(isp - 1), a = IS(isp - 2);
            isp -= 2;
            int r;
            if (op == PET_HIP_EXPR_IADD)
                r = a + b;
            else if (op == PET_HIP_EXPR_ISUB)
                r = a - b;
            else if (op == PET_HIP_EXPR_IMUL)
                r = a * b;
            else if (op == PET_HIP_EXPR_IDIV)
                r = b != 0 ? a / b : 0;
            else
                r = b != 0 ? a % b : 0;
            IS(isp) = r;
            ++isp;
            pc += 1;
            break;
        }
        case PET_HIP_EXPR_LOAD: {
            const int t = c[pc + 1], nd = tab[t];
            const int *shape = c + tab[kMaxTensors + t];
            isp -= nd;
            unsigned off = 0;
            bool inside = true;
            for (int d = 0; d < nd; ++d) {
                const int idx = IS(isp + d);
                const unsigned e = (unsigned)shape[d];
                inside = inside && (unsigned)idx < e;
                off = off * e + (unsigned)idx;
            }
            float v = 0.f;
            if (inside) {
                // the tensor number is the same for every thread: a scalar select
                const float *src = p.in[0];
#pragma unroll
                for (int k = 1; k < kMaxTensors; ++k)
                    src = t == k ? p.in[k] : src;
                v = src[off];
            }
            FS(fsp) = v;
            ++fsp;
            pc += 2;
            break;
        }
        case PET_HIP_EXPR_I2F:
            --isp;
            FS(fsp) = (float)IS(isp);
            ++fsp;
            pc += 1;
            break;
        case PET_HIP_EXPR_FADD:
        case PET_HIP_EXPR_FSUB:
        case PET_HIP_EXPR_FMUL:
        case PET_HIP_EXPR_FDIV:
        case PET_HIP_EXPR_FMOD: {
            const float b = FS(fsp - 1), a = FS(fsp - 2);
            fsp -= 2;
            float r;
            if (op == PET_HIP_EXPR_FADD)
                r = a + b;
            else if (op == PET_HIP_EXPR_FSUB)
                r = a - b;
            else if (op == PET_HIP_EXPR_FMUL)
                r = a * b;
            else if (op == PET_HIP_EXPR_FDIV)
                r = truncf(a / b); // the reference's values are integers
            else
                r = fmodf(a, b);
            FS(fsp) = r;
            ++fsp;
            pc += 1;
            break;
        }
        case PET_HIP_EXPR_FRELU:
            FS(fsp - 1) = fmaxf(FS(fsp - 1), 0.f);
            pc += 1;
            break;
        case PET_HIP_EXPR_FTANH:
            FS(fsp - 1) = tanhf(FS(fsp - 1));
            pc += 1;
            break;
        case PET_HIP_EXPR_RANGE: {
            // nloop, skip, then (slot, left, right, pad) per loop iterator
            const int n = c[pc + 1], skip = c[pc + 2];
            isp -= n;
            bool inside = true;
            for (int d = 0; d < n; ++d) {
                const int *it = c + pc + 3 + 4 * d;
                const int v = IS(isp + d);
                VAR(it[0]) = v;
                inside = inside && v >= it[1] && v < it[2];
            }
            if (inside) {
                pc += 3 + 4 * n;
            } else { // in the padding of the range: its value there is 0
                FS(fsp) = 0.f;
                ++fsp;
                pc = skip;
            }
            break;
        }
        case PET_HIP_EXPR_SUM: {
            // nsum, then (slot, lo, hi) per sum iterator
            const int n = c[pc + 1];
            for (int d = 0; d < n; ++d)
                VAR(c[pc + 2 + 3 * d]) = c[pc + 3 + 3 * d];
            FS(fsp) = 0.f;
            ++fsp;
            pc += 2 + 3 * n;
            break;
        }
        default: { // PET_HIP_EXPR_SUMEND: nsum, body, then (slot, lo, hi) per sum iterator
            const int n = c[pc + 1], body = c[pc + 2];
            --fsp;
            FS(fsp - 1) += FS(fsp);
            // advance the iterators, last one fastest
            int d = n - 1;
            for (; d >= 0; --d) {
                const int *it = c + pc + 3 + 3 * d;
                const int v = VAR(it[0]) + 1;
                if (v < it[2]) {
                    VAR(it[0]) = v;
                    break;
                }
                VAR(it[0]) = it[1];
            }
            pc = d >= 0 ? body : pc + 3 + 3 * n;
            break;
        }
        }
    }
    p.out[i] = FS(fsp - 1);
#undef IS
#undef FS
#undef VAR
}

} // namespace

namespace pet {

// Static check of a program: known opcodes, operands in range, stack depths within the
// interpreter's limits. Fills the per-tensor tables of the launch parameters.
int expr_validate(const int *code, int ncode, int ninputs, int *pc0, int *nd, int *shape_at,
                  size_t *in_elems, int *out_nd, int *out_shape, size_t *out_elems) {
    if (!code || ncode < 4 || code[0] != PET_HIP_EXPR_MAGIC)
        return set_error(PET_HIP_ERR_INVALID, "expr: not a program (bad header)");
    int at = 1;
    const int nt = code[at++];
    if (nt != ninputs || nt < 0 || nt > kMaxTensors)
        return set_error(PET_HIP_ERR_INVALID, "expr: program reads %d tensors, %d given (at most %d)",
                         nt, ninputs, kMaxTensors);
    for (int t = 0; t < nt; ++t) {
        if (at >= ncode)
            return set_error(PET_HIP_ERR_INVALID, "expr: truncated tensor table");
        nd[t] = code[at++];
        if (nd[t] < 0 || nd[t] > PET_HIP_MAX_RANK || at + nd[t] > ncode)
            return set_error(PET_HIP_ERR_INVALID, "expr: bad rank of tensor %d", t);
        shape_at[t] = at;
        size_t n = 1;
        for (int d = 0; d < nd[t]; ++d) {
            if (code[at + d] <= 0)
                return set_error(PET_HIP_ERR_INVALID, "expr: bad extent in tensor %d", t);
            n *= (size_t)code[at + d];
        }
        if (n >= ((size_t)1 << 31))
            return set_error(PET_HIP_ERR_UNSUPPORTED, "expr: tensor %d has 2^31 elements or more", t);
        in_elems[t] = n;
        at += nd[t];
    }
    if (at >= ncode)
        return set_error(PET_HIP_ERR_INVALID, "expr: truncated header");
    *out_nd = code[at++];
    if (*out_nd < 0 || *out_nd > PET_HIP_MAX_RANK || at + *out_nd > ncode)
        return set_error(PET_HIP_ERR_INVALID, "expr: bad output rank");
    *out_elems = 1;
    for (int d = 0; d < *out_nd; ++d) {
        out_shape[d] = code[at + d];
        if (out_shape[d] <= 0)
            return set_error(PET_HIP_ERR_INVALID, "expr: bad output extent");
        *out_elems *= (size_t)out_shape[d];
    }
    at += *out_nd;
    *pc0 = at;
    // one linear pass: operand checks and stack depths (loops leave the depths unchanged)
    int isp = *out_nd, fsp = 0, pc = at;
    bool ended = false;
    auto bad = [&](const char *what) {
        return set_error(PET_HIP_ERR_INVALID, "expr: %s at word %d", what, pc);
    };
    while (pc < ncode) {
        const int op = code[pc];
        int len = 1;
        switch (op) {
        case PET_HIP_EXPR_END:
            ended = true;
            break;
        case PET_HIP_EXPR_ICONST:
            len = 2, ++isp;
            break;
        case PET_HIP_EXPR_IVAR:
            len = 2, ++isp;
            if (pc + 1 >= ncode || code[pc + 1] < 0 || code[pc + 1] >= kMaxVars)
                return bad("bad iterator slot");
            break;
        case PET_HIP_EXPR_IADD:
        case PET_HIP_EXPR_ISUB:
        case PET_HIP_EXPR_IMUL:
        case PET_HIP_EXPR_IDIV:
        case PET_HIP_EXPR_IMOD:
            if (isp < 2)
                return bad("integer stack underflow");
            --isp;
            break;
        case PET_HIP_EXPR_LOAD:
            len = 2;
            if (pc + 1 >= ncode || code[pc + 1] < 0 || code[pc + 1] >= nt)
                return bad("bad tensor number");
            if (isp < nd[code[pc + 1]])
                return bad("integer stack underflow");
            isp -= nd[code[pc + 1]];
            ++fsp;
            break;
        case PET_HIP_EXPR_I2F:
            if (isp < 1)
                return bad("integer stack underflow");
            --isp, ++fsp;
            break;
        case PET_HIP_EXPR_FADD:
        case PET_HIP_EXPR_FSUB:
        case PET_HIP_EXPR_FMUL:
        case PET_HIP_EXPR_FDIV:
        case PET_HIP_EXPR_FMOD:
            if (fsp < 2)
                return bad("value stack underflow");
            --fsp;
            break;
        case PET_HIP_EXPR_FRELU:
        case PET_HIP_EXPR_FTANH:
            if (fsp < 1)
                return bad("value stack underflow");
            break;
        case PET_HIP_EXPR_RANGE: {
            if (pc + 2 >= ncode)
                return bad("truncated range");
            const int n = code[pc + 1], skip = code[pc + 2];
            len = 3 + 4 * n;
            if (n < 0 || n > PET_HIP_MAX_RANK || pc + len > ncode || skip <= pc || skip >= ncode)
                return bad("bad range");
            if (isp < n)
                return bad("integer stack underflow");
            isp -= n;
            for (int d = 0; d < n; ++d)
                if (code[pc + 3 + 4 * d] < 0 || code[pc + 3 + 4 * d] >= kMaxVars)
                    return bad("bad iterator slot");
            break;
        }
        case PET_HIP_EXPR_SUM: {
            if (pc + 1 >= ncode)
                return bad("truncated sum");
            const int n = code[pc + 1];
            len = 2 + 3 * n;
            if (n < 1 || n > PET_HIP_MAX_RANK || pc + len > ncode)
                return bad("bad sum");
            for (int d = 0; d < n; ++d) {
                const int *it = code + pc + 2 + 3 * d;
                if (it[0] < 0 || it[0] >= kMaxVars || it[1] >= it[2])
                    return bad("bad sum iterator");
            }
            ++fsp;
            break;
        }
        case PET_HIP_EXPR_SUMEND: {
            if (pc + 2 >= ncode)
                return bad("truncated sum end");
            const int n = code[pc + 1], body = code[pc + 2];
            len = 3 + 3 * n;
            if (n < 1 || n > PET_HIP_MAX_RANK || pc + len > ncode || body < at || body >= pc)
                return bad("bad sum end");
            for (int d = 0; d < n; ++d) {
                const int *it = code + pc + 3 + 3 * d;
                if (it[0] < 0 || it[0] >= kMaxVars || it[1] >= it[2])
                    return bad("bad sum iterator");
            }
            if (fsp < 2)
                return bad("value stack underflow");
            --fsp;
            break;
        }
        default:
            return bad("unknown opcode");
        }
        if (isp > kStack || fsp > kStack)
            return bad("expression too deep");
        if (ended)
            break;
        pc += len;
    }
    if (!ended || fsp != 1)
        return set_error(PET_HIP_ERR_INVALID, "expr: program does not end with one value");
    return PET_HIP_OK;
}

} // namespace pet

extern "C" {

int pet_hip_expr_program_create(const int *code, int ncode, int **device_code) {
    PET_REQUIRE_INIT();
    if (!device_code)
        return set_error(PET_HIP_ERR_INVALID, "expr: null result pointer");
    int pc0, nd[kMaxTensors], shape_at[kMaxTensors], out_nd, out_shape[PET_HIP_MAX_RANK];
    size_t in_elems[kMaxTensors], out_elems;
    const int nt = code && ncode > 1 ? code[1] : -1;
    if (int rc = expr_validate(code, ncode, nt, &pc0, nd, shape_at, in_elems, &out_nd, out_shape,
                               &out_elems))
        return rc;
    void *buf = nullptr;
    PET_HIP_CHECK(hipMalloc(&buf, (size_t)ncode * sizeof(int)));
    hipError_t e = hipMemcpy(buf, code, (size_t)ncode * sizeof(int), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        (void)hipFree(buf);
        return set_error(PET_HIP_ERR_RUNTIME, "expr: upload of the program failed: %s",
                         hipGetErrorString(e));
    }
    *device_code = static_cast<int *>(buf);
    return PET_HIP_OK;
}

int pet_hip_expr_f32(const int *code, int ncode, const int *device_code,
                     const float *const *inputs, int ninputs, float *out,
                     pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (!device_code || !out || (ninputs > 0 && !inputs))
        return set_error(PET_HIP_ERR_INVALID, "expr: null operand");
    ExprParams p{};
    size_t in_elems[kMaxTensors], out_elems;
    if (int rc = expr_validate(code, ncode, ninputs, &p.pc0, p.nd, p.shape_at, in_elems, &p.out_nd,
                               p.out_shape, &out_elems))
        return rc;
    if (out_elems >= ((size_t)1 << 32))
        return set_error(PET_HIP_ERR_UNSUPPORTED, "expr: output of 2^32 elements or more");
    for (int t = 0; t < ninputs; ++t) {
        if (!inputs[t])
            return set_error(PET_HIP_ERR_INVALID, "expr: null input %d", t);
        p.in[t] = inputs[t];
    }
    p.code = device_code;
    p.ncode = ncode;
    p.out = out;
    p.total = (unsigned)out_elems;
    // small outputs go out as one-wave workgroups so that they still spread over the CUs
    const unsigned nt = out_elems <= 64u * 2048u ? 64u : 256u;
    const unsigned grid = (unsigned)((out_elems + nt - 1) / nt);
    const bool in_lds = ncode <= kMaxLdsCode;
    const size_t lds = sizeof(int) * ((size_t)(2 * kStack + kMaxVars) * nt + 2 * kMaxTensors +
                                      (in_lds ? (size_t)ncode : 0));
    static int attr_status = [] {
        const hipError_t a = hipFuncSetAttribute(reinterpret_cast<const void *>(&expr_kernel<true>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize,
                                                 96 * 1024);
        const hipError_t b = hipFuncSetAttribute(reinterpret_cast<const void *>(&expr_kernel<false>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize,
                                                 96 * 1024);
        return a == hipSuccess && b == hipSuccess ? 0 : 1;
    }();
    if (attr_status)
        return set_error(PET_HIP_ERR_RUNTIME, "expr: cannot size the LDS allocation");
    if (in_lds)
        hipLaunchKernelGGL(expr_kernel<true>, dim3(grid), dim3(nt), lds, as_stream(stream), p);
    else
        hipLaunchKernelGGL(expr_kernel<false>, dim3(grid), dim3(nt), lds, as_stream(stream), p);
    return check_launch("expr_kernel");
}

} // extern "C"
