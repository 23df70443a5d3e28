// Ambient names of the PTO programming model on gfx950: qualifiers, scalar element types, enums, Shape / Stride /
// GlobalTensor.  Reference: include/pto/common/type.hpp:18-23,121-244, common/pto_tile.hpp:32-330,
// common/cpu_stub.hpp:36-61,558-604.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

#ifndef PTO_AMD_THREADS
#define PTO_AMD_THREADS 256  // threads of one core (4 waves)
#endif
// LDS regions (bytes) standing in for the Ascend on-chip buffers (L1, L0A, L0B, UB, bias table, fix-pipe buffer,
// L0 scale buffer, split evenly between the Left and the Right scales); together they must fit the CU's 160 KiB.  Override before including this header.
#ifndef PTO_AMD_L1_BYTES
#define PTO_AMD_L1_BYTES (80 * 1024)
#endif
#ifndef PTO_AMD_L0A_BYTES
#define PTO_AMD_L0A_BYTES (32 * 1024)
#endif
#ifndef PTO_AMD_L0B_BYTES
#define PTO_AMD_L0B_BYTES (32 * 1024)
#endif
#ifndef PTO_AMD_UB_BYTES
#define PTO_AMD_UB_BYTES (8 * 1024)
#endif
#ifndef PTO_AMD_BIAS_BYTES
#define PTO_AMD_BIAS_BYTES (2 * 1024)
#endif
#ifndef PTO_AMD_FB_BYTES
#define PTO_AMD_FB_BYTES (2 * 1024)
#endif
#ifndef PTO_AMD_L0S_BYTES
#define PTO_AMD_L0S_BYTES (4 * 1024)
#endif
// Staging bytes of the fix-pipe (behind the regions above): where TSTORE of an accumulator tile turns the matrix unit's
// register layout into whole rows before they leave for global memory.  A wave stages one 32 x 32 block at a time in a
// band of 32 rows x (row bytes + 16) -- for 16-bit outputs with two blocks side by side in the wave, 16 rows of the
// pair at a time in 16 x (128 + 16) bytes, so that every row leaves as a whole 128-byte line; with fewer bytes than
// WAVES such bands of the output type, TSTORE writes each lane's register quads directly (8 or 16 bytes per row and
// store).  0 by default: the default split of the other regions already fills the CU's 160 KiB.
#ifndef PTO_AMD_STAGE_BYTES
#define PTO_AMD_STAGE_BYTES 0
#endif
// PTO_AMD_TLOAD_AFTER_ACQUIRE (defined by the kernel source, off by default): a promise about program order that saves
// the asynchronous TLOAD its own workgroup barrier.  Before it overwrites a Mat tile, TLOAD must know that no wave is
// still reading the tile's old contents -- directly, or through Left / Right / scale windows in a TMATMUL.  By default it
// runs a barrier of its own.  With the macro defined the kernel promises that, between the last instruction that read
// the tile and the TLOAD, every core executes an instruction that waits for a pending load (the first TEXTRACT / TMOV /
// TSTORE of any freshly loaded tile: that wait ends in a barrier).  The double-buffered order of the reference's
// kernels -- TEXTRACT(panel p) ... TLOAD(panel p + 1 into the other buffer) ... TMATMUL(panel p) -- keeps the promise:
// the other buffer's last readers were the TMATMULs of panel p - 1, before the TEXTRACT of panel p waited for its load.
// It is what the reference writes as wait_flag(PIPE_MTE1, PIPE_MTE2) in front of such a TLOAD.

// A PTO kernel entry is written `__global__ AICORE void f(...)`; here it is a device function run by pto::amd::launch.
// (PTO_AMD_CHECK_REFERENCE_SOURCE: a device-only syntax pass over an unmodified reference kernel file, whose
// CPU-simulator launch functions call the core programs directly; the cores are then also callable from host code.)
#undef __global__
#define __global__
#ifdef PTO_AMD_CHECK_REFERENCE_SOURCE
#define AICORE __host__ __device__
#else
#define AICORE __device__
#endif
#define __aicore__
#define __gm__
#define __ubuf__
#define __cbuf__
#define __ca__
#define __cb__
#define __cc__
#define __fbuf__
#define __tf__
#define __in__
#define __out__
#define PTO_INST __device__ __forceinline__
#define PTO_INTERNAL __device__ __forceinline__

using half = _Float16;
using aclFloat16 = _Float16;
using bfloat16_t = __bf16;

namespace pto {

// one-byte MX element types (storage only; arithmetic happens in the MFMA or after decode)
struct float8_e4m3_t { uint8_t raw; };
struct float8_e5m2_t { uint8_t raw; };
struct float8_e8m0_t { uint8_t raw; };
struct float4_e2m1x2_t { uint8_t raw; };  // two codes per byte, even element in the low nibble
struct float4_e1m2x2_t { uint8_t raw; };

constexpr int DYNAMIC = -1;

enum class TileType { Vec, Mat, Left, Right, Acc, Bias, Scaling, ScaleLeft, ScaleRight, Ctrl };
enum class BLayout { RowMajor = 0, ColMajor = 1 };
enum class SLayout { NoneBox = 0, RowMajor = 1, ColMajor = 2 };
enum class Layout { ND, DN, NZ, SCALE, MX_A_ND, MX_A_DN, MX_A_ZZ, MX_B_ND, MX_B_DN, MX_B_NN };
enum class PadValue { Null, Zero, Max, Min };
enum class CompactMode { Null, Normal };
enum class AtomicType { AtomicNone = 0, AtomicAdd = 1 };
enum class ReluPreMode { NoRelu = 0, NormalRelu = 1 };
enum class AccPhase : uint8_t { Unspecified = 0, Unknown = 0, Partial = 2, Final = 3 };
enum class STPhase : uint8_t { Unspecified = 0, Partial = 2, Final = 3 };

struct TileConfig {
    static constexpr int alignedSize = 32, fixedRowSize = 16, fixedColSize = 16, fixedMxRowSize = 16, fixedMxColSize = 2;
    static constexpr int fractalABSize = 512, fractalCSize = 1024, fractalMxSize = 32;
};

struct GlobalTensorDim {
    static constexpr int DIM_0 = 0, DIM_1 = 1, DIM_2 = 2, DIM_3 = 3, DIM_4 = 4, TOTAL_DIM = 5;
};

// Shape<N1..N5> / Stride<S1..S5>: static extents, DYNAMIC ones supplied to the constructor in order.
template <int64_t N1 = DYNAMIC, int64_t N2 = DYNAMIC, int64_t N3 = DYNAMIC, int64_t N4 = DYNAMIC, int64_t N5 = DYNAMIC>
struct Shape {
    static constexpr int64_t staticShape[5] = {N1, N2, N3, N4, N5};
    int64_t shape[5] = {N1, N2, N3, N4, N5};
    __host__ __device__ constexpr Shape() {}
    template <typename... D, typename = std::enable_if_t<(sizeof...(D) > 0)>>
    __host__ __device__ constexpr Shape(D... dyn)
    {
        const int64_t v[] = {static_cast<int64_t>(dyn)...};
        int next = 0;
        for (int i = 0; i < 5; ++i)
            if (staticShape[i] == DYNAMIC && next < (int)sizeof...(D))
                shape[i] = v[next++];
    }
};
template <int64_t S1 = DYNAMIC, int64_t S2 = DYNAMIC, int64_t S3 = DYNAMIC, int64_t S4 = DYNAMIC, int64_t S5 = DYNAMIC>
struct Stride {
    static constexpr int64_t staticStride[5] = {S1, S2, S3, S4, S5};
    int64_t stride[5] = {S1, S2, S3, S4, S5};
    __host__ __device__ constexpr Stride() {}
    template <typename... D, typename = std::enable_if_t<(sizeof...(D) > 0)>>
    __host__ __device__ constexpr Stride(D... dyn)
    {
        const int64_t v[] = {static_cast<int64_t>(dyn)...};
        int next = 0;
        for (int i = 0; i < 5; ++i)
            if (staticStride[i] == DYNAMIC && next < (int)sizeof...(D))
                stride[i] = v[next++];
    }
};

// A view of global memory: element type, 5-D shape and strides (in elements), and how a tile's (row, col) walks the
// dimensions (Layout).  Reference: common/pto_tile.hpp:276-330, index maps cpu/tile_offsets.hpp:181-277.
template <typename Element_, typename Shape_, typename Stride_, Layout Layout_ = Layout::ND>
struct GlobalTensor {
    using Shape = Shape_;
    using Stride = Stride_;
    using RawDType = std::remove_cv_t<Element_>;
    using DType = RawDType;
    static constexpr Layout layout = Layout_;
    __host__ __device__ GlobalTensor(DType* data, const Shape& shape = Shape{}, const Stride& stride = Stride{})
        : data_(data), shape_(shape), stride_(stride)
    {
    }
    __host__ __device__ DType* data() const { return data_; }
    __host__ __device__ int64_t GetShape(int dim) const { return shape_.shape[dim]; }
    __host__ __device__ int64_t GetStride(int dim) const { return stride_.stride[dim]; }
    // element offset of logical (r, c)
    __host__ __device__ int64_t Offset(int64_t r, int64_t c) const
    {
        const int64_t* sh = shape_.shape;
        const int64_t* st = stride_.stride;
        int64_t i0, i1, i2, i3, i4;
        if constexpr (Layout_ == Layout::DN) {
            i3 = r;
            i4 = c % sh[4];
            i2 = (c / sh[4]) % sh[2];
            i1 = (c / (sh[4] * sh[2])) % sh[1];
            i0 = c / (sh[1] * sh[2] * sh[4]);
        } else if constexpr (Layout_ == Layout::NZ) {
            const int64_t outer = c / sh[4];
            i0 = outer / sh[1];
            i1 = outer % sh[1];
            i2 = r / sh[3];
            i3 = r % sh[3];
            i4 = c % sh[4];
        } else if constexpr (Layout_ == Layout::MX_A_ZZ) {  // E8M0 scales of the A side: r = row, c = K-group
            i0 = 0; i1 = r / 16; i2 = c / 2; i3 = r % 16; i4 = c % 2;
        } else if constexpr (Layout_ == Layout::MX_B_NN) {  // B side: r = K-group, c = column
            i0 = 0; i1 = c / 16; i2 = r / 2; i3 = c % 16; i4 = r % 2;
        } else if constexpr (Layout_ == Layout::MX_A_ND) {
            i0 = 0; i1 = 0; i2 = r; i3 = c / 2; i4 = c % 2;
        } else if constexpr (Layout_ == Layout::MX_A_DN) {
            i0 = 0; i1 = 0; i2 = c / 2; i3 = r; i4 = c % 2;
        } else if constexpr (Layout_ == Layout::MX_B_ND) {
            i0 = 0; i1 = 0; i2 = r / 2; i3 = c; i4 = r % 2;
        } else if constexpr (Layout_ == Layout::MX_B_DN) {
            i0 = 0; i1 = 0; i2 = c; i3 = r / 2; i4 = r % 2;
        } else {
            static_assert(Layout_ == Layout::ND, "GlobalTensor layout not supported by the gfx950 backend");
            i4 = c;
            i3 = r % sh[3];
            i2 = (r / sh[3]) % sh[2];
            i1 = (r / (sh[3] * sh[2])) % sh[1];
            i0 = r / (sh[1] * sh[2] * sh[3]);
        }
        return i0 * st[0] + i1 * st[1] + i2 * st[2] + i3 * st[3] + i4 * st[4];
    }
    // logical 2-D extent a tile sees
    __host__ __device__ int64_t Rows() const
    {
        const int64_t* sh = shape_.shape;
        if constexpr (Layout_ == Layout::DN)
            return sh[3];
        else if constexpr (Layout_ == Layout::NZ)
            return sh[2] * sh[3];
        else
            return sh[0] * sh[1] * sh[2] * sh[3];
    }
    __host__ __device__ int64_t Cols() const
    {
        const int64_t* sh = shape_.shape;
        if constexpr (Layout_ == Layout::DN)
            return sh[0] * sh[1] * sh[2] * sh[4];
        else if constexpr (Layout_ == Layout::NZ)
            return sh[0] * sh[1] * sh[4];
        else
            return sh[4];
    }

private:
    DType* data_;
    Shape shape_;
    Stride stride_;
};

// Shape / stride of a whole [rows, cols] logical matrix in a given layout (reference: common/pto_tile.hpp:664-1101).
// BaseShape2D is the *stride* type, as in the reference.  For the MX layouts rows x cols is the logical scale matrix
// ([M][K/32] on the A side, [K/32][N] on the B side).
template <typename T, int64_t rows, int64_t cols, Layout L = Layout::ND>
struct TileShape2D;
template <typename T, int64_t rows, int64_t cols, Layout L = Layout::ND>
struct BaseShape2D;
#define PTO_AMD_SHAPE2D(LAYOUT, SHAPE, STRIDE)                                          \
    template <typename T, int64_t rows, int64_t cols>                                 \
    struct TileShape2D<T, rows, cols, LAYOUT> : SHAPE {                               \
        using Parent = SHAPE;                                                         \
        using Parent::Parent;                                                         \
    };                                                                                \
    template <typename T, int64_t rows, int64_t cols>                                 \
    struct BaseShape2D<T, rows, cols, LAYOUT> : STRIDE {                              \
        using Parent = STRIDE;                                                        \
        using Parent::Parent;                                                         \
    };
#define PTO_AMD_C(...) __VA_ARGS__
PTO_AMD_SHAPE2D(Layout::ND, PTO_AMD_C(Shape<1, 1, 1, rows, cols>), PTO_AMD_C(Stride<rows * cols, rows * cols, rows * cols, cols, 1>))
PTO_AMD_SHAPE2D(Layout::DN, PTO_AMD_C(Shape<1, 1, 1, rows, cols>), PTO_AMD_C(Stride<rows * cols, rows * cols, rows * cols, 1, rows>))
// NZ: column blocks of C0 = 32 bytes' worth of elements, rows contiguous inside a block (reference: pto_tile.hpp:709-725,797-815)
PTO_AMD_SHAPE2D(Layout::NZ, PTO_AMD_C(Shape<1, cols / (32 / (int64_t)sizeof(T)), rows / 16, 16, 32 / (int64_t)sizeof(T)>),
                PTO_AMD_C(Stride<rows * cols, rows * (32 / (int64_t)sizeof(T)), 16 * (32 / (int64_t)sizeof(T)), 32 / (int64_t)sizeof(T), 1>))
PTO_AMD_SHAPE2D(Layout::MX_A_ZZ, PTO_AMD_C(Shape<1, rows / 16, cols / 2, 16, 2>), PTO_AMD_C(Stride<rows * cols, cols * 16, 32, 2, 1>))
PTO_AMD_SHAPE2D(Layout::MX_A_ND, PTO_AMD_C(Shape<1, 1, rows, cols / 2, 2>), PTO_AMD_C(Stride<rows * cols, rows * cols, cols, 2, 1>))
PTO_AMD_SHAPE2D(Layout::MX_A_DN, PTO_AMD_C(Shape<1, 1, cols / 2, rows, 2>), PTO_AMD_C(Stride<rows * cols, rows * cols, 2 * rows, 2, 1>))
PTO_AMD_SHAPE2D(Layout::MX_B_NN, PTO_AMD_C(Shape<1, cols / 16, rows / 2, 16, 2>), PTO_AMD_C(Stride<rows * cols, rows * 16, 32, 2, 1>))
PTO_AMD_SHAPE2D(Layout::MX_B_ND, PTO_AMD_C(Shape<1, 1, rows / 2, cols, 2>), PTO_AMD_C(Stride<rows * cols, rows * cols, 2 * cols, 2, 1>))
PTO_AMD_SHAPE2D(Layout::MX_B_DN, PTO_AMD_C(Shape<1, 1, cols, rows / 2, 2>), PTO_AMD_C(Stride<rows * cols, rows * cols, rows, 2, 1>))
#undef PTO_AMD_SHAPE2D
#undef PTO_AMD_C

// ---- pipes and event ids (reference: common/cpu_stub.hpp:36-61): names only, ordering is by workgroup barriers
using pipe_t = int;
using event_t = int;
}  // namespace pto

constexpr pto::pipe_t PIPE_S = 0, PIPE_V = 1, PIPE_M = 2, PIPE_MTE1 = 3, PIPE_MTE2 = 4, PIPE_MTE3 = 5, PIPE_ALL = 6,
                      PIPE_FIX = 7;
constexpr pto::event_t EVENT_ID0 = 0, EVENT_ID1 = 1, EVENT_ID2 = 2, EVENT_ID3 = 3, EVENT_ID4 = 4, EVENT_ID5 = 5,
                       EVENT_ID6 = 6, EVENT_ID7 = 7;
PTO_INST void set_flag(pto::pipe_t, pto::pipe_t, pto::event_t) {}
PTO_INST void wait_flag(pto::pipe_t, pto::pipe_t, pto::event_t) {}
PTO_INST void pipe_barrier(pto::pipe_t) { __syncthreads(); }
PTO_INST int64_t get_block_idx() { return blockIdx.x; }
PTO_INST int64_t get_block_num() { return gridDim.x; }
PTO_INST int64_t get_subblockid() { return 0; }

using pto::float4_e1m2x2_t;
using pto::float4_e2m1x2_t;
using pto::float8_e4m3_t;
using pto::float8_e5m2_t;
using pto::float8_e8m0_t;
