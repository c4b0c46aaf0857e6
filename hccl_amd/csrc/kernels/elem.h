// Element arithmetic of the reduce kernels: one functor per HcclDataType x HcclReduceOp.
//
// Every reduction is applied as  dst = src (+) dst  with the operand order of the reference's scalar loop
// AicpuReduceTemplate (src/ops/op_common/template/wrapper/alg_data_trans_wrapper.cc:1221-1250):
//   SUM  : src + dst           PROD : src * dst  (integers through unsigned wrap-around, :1229-1234)
//   MAX  : std::max(src, dst) == (src < dst) ? dst : src
//   MIN  : std::min(src, dst) == (dst < src) ? dst : src
// fp16 follows AicpuReduceFp16 (:1140-1163): widen both operands to fp32, operate, narrow with
// round-to-nearest-even.  For a single pairwise step that equals the correctly rounded half-precision
// result, so the hardware conversions are used.  bf16 has no CPU path in the reference (its reduce runs
// in HCOMM hardware); it is defined here the same way: fp32 arithmetic, one RNE narrowing.
//
// In a fused N-way fold the 16-bit float SUM keeps its accumulator in fp32 and narrows once at the end
// (the "fp32-accumulated result"); PROD narrows after every step, because that is what the reference's
// CPU path does for fp16 PROD.  MAX/MIN only select, so no rounding is involved.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "hccl_types.h"

namespace hcclx {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// A 16-byte vector that may sit at any byte address.  gfx950 global loads/stores accept that, and the
// compiler keeps them as one dwordx4 access.
typedef u32x4 u32x4_u __attribute__((aligned(1)));

template <typename T> struct UnsignedOf { using type = T; };
template <> struct UnsignedOf<int8_t> { using type = uint8_t; };
template <> struct UnsignedOf<int16_t> { using type = uint16_t; };
template <> struct UnsignedOf<int32_t> { using type = uint32_t; };
template <> struct UnsignedOf<int64_t> { using type = uint64_t; };

__device__ __forceinline__ float bf16_widen(uint16_t b)
{
    return __uint_as_float(static_cast<uint32_t>(b) << 16);
}

__device__ __forceinline__ uint16_t bf16_narrow(float f)
{
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        return static_cast<uint16_t>((u >> 16) | 0x0040u);  // NaN stays NaN (quiet bit forced)
    }
    u += 0x7fffu + ((u >> 16) & 1u);  // round to nearest, ties to even; overflow carries into Inf
    return static_cast<uint16_t>(u >> 16);
}

__device__ __forceinline__ float fp16_widen(uint16_t h)
{
    _Float16 x;
    __builtin_memcpy(&x, &h, 2);
    return static_cast<float>(x);
}

__device__ __forceinline__ uint16_t fp16_narrow(float f)
{
    _Float16 x = static_cast<_Float16>(f);
    uint16_t h;
    __builtin_memcpy(&h, &x, 2);
    return h;
}

// Storage type S (what sits in memory) and compute type C (what the fold runs in).
template <int DT> struct DTypeOf;
#define HCCLX_PLAIN_DTYPE(DT, T)                                                  \
    template <> struct DTypeOf<DT> {                                              \
        using S = T;                                                              \
        using C = T;                                                              \
        static constexpr bool kHalfFloat = false;                                 \
        static __device__ __forceinline__ C widen(S s) { return s; }              \
        static __device__ __forceinline__ S narrow(C c) { return c; }             \
    };
HCCLX_PLAIN_DTYPE(HCCL_DATA_TYPE_INT8, int8_t)
HCCLX_PLAIN_DTYPE(HCCL_DATA_TYPE_INT16, int16_t)
HCCLX_PLAIN_DTYPE(HCCL_DATA_TYPE_INT32, int32_t)
HCCLX_PLAIN_DTYPE(HCCL_DATA_TYPE_INT64, int64_t)
HCCLX_PLAIN_DTYPE(HCCL_DATA_TYPE_UINT64, uint64_t)
HCCLX_PLAIN_DTYPE(HCCL_DATA_TYPE_FP32, float)
HCCLX_PLAIN_DTYPE(HCCL_DATA_TYPE_FP64, double)
#undef HCCLX_PLAIN_DTYPE

template <> struct DTypeOf<HCCL_DATA_TYPE_FP16> {
    using S = uint16_t;
    using C = float;
    static constexpr bool kHalfFloat = true;
    static __device__ __forceinline__ C widen(S s) { return fp16_widen(s); }
    static __device__ __forceinline__ S narrow(C c) { return fp16_narrow(c); }
};

template <> struct DTypeOf<HCCL_DATA_TYPE_BFP16> {
    using S = uint16_t;
    using C = float;
    static constexpr bool kHalfFloat = true;
    static __device__ __forceinline__ C widen(S s) { return bf16_widen(s); }
    static __device__ __forceinline__ S narrow(C c) { return bf16_narrow(c); }
};

// src (+) dst on the compute type.
template <int DT, int OP> struct Combine {
    using D = DTypeOf<DT>;
    using C = typename D::C;
    static __device__ __forceinline__ C run(C s, C d)
    {
        if constexpr (OP == HCCL_REDUCE_MAX) {
            return (s < d) ? d : s;
        } else if constexpr (OP == HCCL_REDUCE_MIN) {
            return (d < s) ? d : s;
        } else if constexpr (__is_integral(C)) {
            using U = typename UnsignedOf<C>::type;
            if constexpr (OP == HCCL_REDUCE_SUM) {
                return static_cast<C>(static_cast<U>(static_cast<U>(s) + static_cast<U>(d)));
            } else {
                return static_cast<C>(static_cast<U>(static_cast<U>(s) * static_cast<U>(d)));
            }
        } else if constexpr (OP == HCCL_REDUCE_SUM) {
            return s + d;
        } else {
            C p = s * d;
            if constexpr (D::kHalfFloat) {
                p = D::widen(D::narrow(p));  // the CPU path narrows after every product
            }
            return p;
        }
    }
};

// 16 bytes of storage elements <-> compute-type registers.
template <int DT> struct Vec16 {
    using D = DTypeOf<DT>;
    using S = typename D::S;
    using C = typename D::C;
    static constexpr int NE = 16 / static_cast<int>(sizeof(S));   // compute registers per 16 bytes
    static constexpr int kElems = NE;                             // elements per 16 bytes

    static __device__ __forceinline__ void unpack(u32x4 raw, C (&out)[NE])
    {
        S tmp[NE];
        __builtin_memcpy(tmp, &raw, 16);
#pragma unroll
        for (int e = 0; e < NE; ++e) out[e] = D::widen(tmp[e]);
    }

    static __device__ __forceinline__ u32x4 pack(const C (&in)[NE])
    {
        S tmp[NE];
#pragma unroll
        for (int e = 0; e < NE; ++e) tmp[e] = D::narrow(in[e]);
        u32x4 raw;
        __builtin_memcpy(&raw, tmp, 16);
        return raw;
    }

    template <int OP> static __device__ __forceinline__ C combine(C s, C d) { return Combine<DT, OP>::run(s, d); }
};

// int8 stays packed, four elements to a 32-bit register: byte-wise arithmetic element by element costs
// several instructions per byte and makes the fold compute-bound.
typedef short i16x2 __attribute__((ext_vector_type(2)));
template <> struct Vec16<HCCL_DATA_TYPE_INT8> {
    using D = DTypeOf<HCCL_DATA_TYPE_INT8>;
    using S = int8_t;
    using C = uint32_t;   // four int8
    static constexpr int NE = 4;
    static constexpr int kElems = 16;

    static __device__ __forceinline__ void unpack(u32x4 raw, C (&out)[NE])
    {
        out[0] = raw.x;
        out[1] = raw.y;
        out[2] = raw.z;
        out[3] = raw.w;
    }
    static __device__ __forceinline__ u32x4 pack(const C (&in)[NE])
    {
        u32x4 raw = {in[0], in[1], in[2], in[3]};
        return raw;
    }

    template <int OP> static __device__ __forceinline__ C combine(C s, C d)
    {
        if constexpr (OP == HCCL_REDUCE_SUM) {
            // add the low 7 bits of every byte, then put the top bits back without carrying across bytes
            return ((s & 0x7f7f7f7fu) + (d & 0x7f7f7f7fu)) ^ ((s ^ d) & 0x80808080u);
        } else if constexpr (OP == HCCL_REDUCE_PROD) {
            C r = 0;
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                r |= (((s >> (8 * b)) & 0xffu) * ((d >> (8 * b)) & 0xffu) & 0xffu) << (8 * b);
            }
            return r;
        } else {
            // A byte in the high half of a 16-bit lane orders like the signed byte itself: even bytes are
            // shifted up, odd bytes are already there; two packed 16-bit max/min cover all four.
            const C se = (s << 8) & 0xff00ff00u;
            const C de = (d << 8) & 0xff00ff00u;
            const C so = s & 0xff00ff00u;
            const C dp = d & 0xff00ff00u;
            i16x2 a, b, c, e;
            __builtin_memcpy(&a, &se, 4);
            __builtin_memcpy(&b, &de, 4);
            __builtin_memcpy(&c, &so, 4);
            __builtin_memcpy(&e, &dp, 4);
            i16x2 me, mo;
            if constexpr (OP == HCCL_REDUCE_MAX) {
                me = __builtin_elementwise_max(a, b);
                mo = __builtin_elementwise_max(c, e);
            } else {
                me = __builtin_elementwise_min(a, b);
                mo = __builtin_elementwise_min(c, e);
            }
            C ue, uo;
            __builtin_memcpy(&ue, &me, 4);
            __builtin_memcpy(&uo, &mo, 4);
            return (ue >> 8) | uo;
        }
    }
};

// Floating-point max and min select one operand, so  a (+) b  and  b (+) a  differ for signed zeros and NaNs;
// every other type and op gives the same bits either way.
template <int DT, int OP> struct OperandOrderMatters {
    static constexpr bool value =
        (OP == HCCL_REDUCE_MAX || OP == HCCL_REDUCE_MIN) &&
        (DT == HCCL_DATA_TYPE_FP16 || DT == HCCL_DATA_TYPE_FP32 || DT == HCCL_DATA_TYPE_FP64 || DT == HCCL_DATA_TYPE_BFP16);
};

__host__ __device__ constexpr int dtype_size(int dt)
{
    // DATATYPE_SIZE_TABLE, src/ops/op_common/inc/alg_param.h:43-45
    constexpr int t[18] = {1, 2, 4, 2, 4, 8, 8, 1, 2, 4, 8, 2, 16, 2, 1, 1, 1, 1};
    return (dt >= 0 && dt < 18) ? t[dt] : 0;
}

}  // namespace hcclx
