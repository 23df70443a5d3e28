// Per-instruction trace of PTO core programs, the counterpart of the simulator's PtoInstrTraceScope / trace.jsonl
// (reference: include/pto/cpu/trace.hpp:67-153, include/pto/common/pto_instr.hpp:32-68).
//
// A build mode, like the reference's (its scopes exist under __CPU_SIM only): a translation unit compiled with
// -DPTO_AMD_TRACE gets a record per executed tile instruction -- opcode, output and input operands with address, shape,
// layout and dtype -- written by thread 0 of one core (PTO_AMD_TRACE_CORE, default core 0) into a device buffer of
// PTO_AMD_TRACE_MAX records; pto::amd::launch then waits for the kernel, reads the buffer back and appends one JSON line
// per record to $PTOAMD_TRACE_DIR/ptoamd_instr_trace_<pid>.jsonl (nothing is written when the variable is unset).
// Without the macro none of this exists in the compiled kernels.
#pragma once
#include "tile.hpp"

#ifdef PTO_AMD_TRACE
#ifndef PTO_AMD_TRACE_MAX
#define PTO_AMD_TRACE_MAX 4096
#endif
#ifndef PTO_AMD_TRACE_CORE
#define PTO_AMD_TRACE_CORE 0
#endif

namespace pto {
namespace amd {

enum TraceOp : uint16_t {
    TR_TLOAD, TR_TSTORE, TR_TSTORE_FP, TR_TMOV, TR_TEXTRACT, TR_TMATMUL, TR_TMATMUL_ACC, TR_TMATMUL_BIAS, TR_TMATMUL_MX, TR_TGEMV,
    TR_TGEMV_ACC, TR_TGEMV_BIAS, TR_TGEMV_MX, TR_TQUANT, TR_TDEQUANT, TR_TCVT, TR_TFILLPAD, TR_TRESHAPE, TR_COUNT
};
inline const char* trace_op_name(int op)
{
    static const char* const names[TR_COUNT] = {"TLOAD", "TSTORE", "TSTORE_FP", "TMOV", "TEXTRACT", "TMATMUL", "TMATMUL_ACC",
                                                "TMATMUL_BIAS", "TMATMUL_MX", "TGEMV", "TGEMV_ACC", "TGEMV_BIAS", "TGEMV_MX", "TQUANT",
                                                "TDEQUANT", "TCVT", "TFILLPAD", "TRESHAPE"};
    return op >= 0 && op < TR_COUNT ? names[op] : "?";
}
// element types, in the reference's spelling (TraceDTypeName, cpu/trace.hpp:241-300)
enum TraceDType : uint8_t { TD_F32, TD_F16, TD_BF16, TD_I32, TD_I16, TD_I8, TD_U8, TD_U64, TD_E4M3, TD_E5M2, TD_E8M0, TD_E2M1X2, TD_E1M2X2, TD_OTHER };
inline const char* trace_dtype_name(int t)
{
    static const char* const names[] = {"float32", "float16", "bfloat16", "int32", "int16", "int8", "uint8", "uint64", "float8_e4m3",
                                        "float8_e5m2", "float8_e8m0", "float4_e2m1x2", "float4_e1m2x2", "other"};
    return t >= 0 && t <= TD_OTHER ? names[t] : "other";
}
template <typename T>
constexpr uint8_t trace_dtype()
{
    using D = std::remove_cv_t<T>;
    return std::is_same_v<D, float>              ? TD_F32
           : std::is_same_v<D, _Float16>         ? TD_F16
           : std::is_same_v<D, __bf16>           ? TD_BF16
           : std::is_same_v<D, int32_t>          ? TD_I32
           : std::is_same_v<D, int16_t>          ? TD_I16
           : std::is_same_v<D, int8_t>           ? TD_I8
           : std::is_same_v<D, uint8_t>          ? TD_U8
           : std::is_same_v<D, uint64_t>         ? TD_U64
           : std::is_same_v<D, float8_e4m3_t>    ? TD_E4M3
           : std::is_same_v<D, float8_e5m2_t>    ? TD_E5M2
           : std::is_same_v<D, float8_e8m0_t>    ? TD_E8M0
           : std::is_same_v<D, float4_e2m1x2_t>  ? TD_E2M1X2
           : std::is_same_v<D, float4_e1m2x2_t>  ? TD_E1M2X2
                                                 : TD_OTHER;
}
// where an operand lives: the tile types, then the global-tensor layouts
inline const char* trace_place_name(int p)
{
    static const char* const names[] = {"Vec", "Mat", "Left", "Right", "Acc", "Bias", "Scaling", "ScaleLeft", "ScaleRight", "Ctrl",
                                        "ND", "DN", "NZ", "SCALE", "MX_A_ND", "MX_A_DN", "MX_A_ZZ", "MX_B_ND", "MX_B_DN", "MX_B_NN"};
    return p >= 0 && p < 20 ? names[p] : "?";
}

struct TraceOperand {
    uint64_t address;  // a tile's TASSIGN address inside its buffer, a global tensor's device address
    int32_t rows, cols;
    uint8_t place, dtype, used, pad;
};
struct TraceRecord {
    uint32_t block_idx;
    uint16_t opcode, n_out;
    TraceOperand operands[4];  // outputs first
};
static __device__ TraceRecord g_trace[PTO_AMD_TRACE_MAX];
static __device__ unsigned int g_trace_count = 0;

template <typename T>
PTO_INST TraceOperand trace_operand(const T& x)
{
    TraceOperand o{};
    o.used = 1;
    if constexpr (is_tile_data_v<T>) {
        o.address = x.data();
        o.rows = x.GetValidRow();
        o.cols = x.GetValidCol();
        o.place = (uint8_t)T::Loc;
        o.dtype = trace_dtype<typename T::DType>();
    } else {  // a GlobalTensor
        o.address = reinterpret_cast<uint64_t>(x.data());
        o.rows = (int32_t)x.Rows();
        o.cols = (int32_t)x.Cols();
        o.place = (uint8_t)(10 + (int)T::layout);
        o.dtype = trace_dtype<typename T::DType>();
    }
    return o;
}
// record one instruction: the first n_out operands are outputs
template <int N_OUT, typename... Ts>
PTO_INST void trace_instr(TraceOp op, const Ts&... xs)
{
    static_assert(sizeof...(Ts) <= 4, "a trace record holds four operands");
    if (threadIdx.x == 0 && blockIdx.x == PTO_AMD_TRACE_CORE) {
        const unsigned int i = atomicAdd(&g_trace_count, 1u);
        if (i < PTO_AMD_TRACE_MAX) {
            TraceRecord r{};
            r.block_idx = blockIdx.x;
            r.opcode = (uint16_t)op;
            r.n_out = N_OUT;
            int k = 0;
            ((r.operands[k++] = trace_operand(xs)), ...);
            g_trace[i] = r;
        }
    }
}

}  // namespace amd
}  // namespace pto
#define PTO_AMD_TRACE_INSTR(N_OUT, OP, ...) ::pto::amd::trace_instr<N_OUT>(::pto::amd::OP, __VA_ARGS__)
// an opcode handed down as a template argument (one body serves TMATMUL_MX and TGEMV_MX)
#define PTO_AMD_TR(OP) ::pto::amd::OP
#define PTO_AMD_TRACE_OP(OP) TraceOp(OP)
namespace pto { namespace amd { using TraceOpOrInt = int; } }
#else
#define PTO_AMD_TRACE_INSTR(N_OUT, OP, ...)
#define PTO_AMD_TR(OP) 0
#define PTO_AMD_TRACE_OP(OP) OP
namespace pto { namespace amd { using TraceOpOrInt = int; } }
#endif
