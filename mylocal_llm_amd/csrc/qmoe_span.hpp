// Single-token weight streaming through LDS: the rows of a packed matrix travel from HBM to a
// wave-private ring of LDS slots as whole spans (consecutive lanes fetch consecutive 16 bytes
// with global_load_lds_dwordx4, so every cache line is requested once, by one instruction, and
// no register holds a byte in flight), and each lane then reads its own 64-element unit of the
// span from LDS, decodes it in registers and accumulates in fp32.  The memory pipeline is fed by
// the ring, not by the number of waves: a wave requests the span of a later item, then waits for
// the oldest one (s_waitcnt vmcnt with the number of newer requests) and multiplies it.
//
// LDS image of a span, per four 64-element units (= 256 columns):
//   Q8_0  272 B = 17 pieces, the bytes as they lie in memory (rows of K % 256 == 0 are 16-byte multiples)
//   Q5_K  176 B = 11 pieces, one block as it lies
//   Q4_K  144 B =  9 pieces, one block as it lies
//   Q6_K  224 B = 14 pieces for a 210-byte block: pieces 0..12 are bytes 0..207, piece 13 is bytes
//         194..209 (so nothing past the block is read and every block starts 16-byte aligned in
//         LDS whatever its alignment in memory); d lies at image byte 222
#pragma once
#include "qmoe_stream.hpp"

namespace qmoe {

static constexpr int SPAN_WAVES = 8;                 // one workgroup of eight waves per CU
static constexpr int SPAN_THREADS = SPAN_WAVES * 64;
static constexpr int SPAN_MAX_KEYS = STREAM_MAX_PROBLEMS;

template <int N> __device__ __forceinline__ void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4) | (0xF << 8));
    asm volatile("" ::: "memory");
}

// 16 bytes per lane from global memory straight into LDS: lane l's piece lands at LDS byte
// m0 + OFFSET + 16 l and is read from base + voff + OFFSET (the immediate offset moves both
// sides).  Inline assembly on purpose: the compiler would order every later LDS read behind ALL
// outstanding requests of a load it knows to write LDS; the waits are this file's own.
#define QMOE_DMA16(base, voff, OFFSET) \
    asm volatile("global_load_lds_dwordx4 %0, %1 offset:" #OFFSET :: "v"(voff), "s"(uniform((const uint8_t*)(base))) : "memory")
// (Two wait-state rules of the ISA manual that the compiler keeps for its own instructions are NOT
// kept around this inline assembly, which its hazard recogniser does not look into: one wait state
// between a scalar write of M0 and an LDS-DMA that reads it (back to back in the whole-slot request
// of span_kernel), and five between a vector instruction that writes a scalar register
// (v_readfirstlane, what uniform() becomes when the value lives in vector registers: the base of a
// gate/up pair's request) and a memory instruction that reads it as its base.  Every result of
// those requests has been right on MI355X, where the hardware evidently settles both; the
// by-the-book form is an "s_nop 0" behind the s_mov below and an "s_nop 4" ahead of a load whose
// base was just made uniform, at the price of issue slots in the streaming loop.)
__device__ __forceinline__ void set_m0(uint32_t v) { asm volatile("s_mov_b32 m0, %0" :: "s"(uniform((int)v)) : "memory"); }
// the same on the lanes of `mask` only (a wave-uniform 64-bit lane mask, not zero)
__device__ __forceinline__ void dma16_masked(const void* base, uint32_t voff, uint64_t mask) {
    uint64_t save;
    mask = ((uint64_t)(uint32_t)uniform((int)(mask >> 32)) << 32) | (uint32_t)uniform((int)(uint32_t)mask);
    asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, %3\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b64 exec, %0"
                 : "=&s"(save) : "v"(voff), "s"(uniform((const uint8_t*)base)), "s"(mask) : "memory");
}

// Activations in LDS as fp32: 16-byte granules XOR-swizzled inside groups of 16 64-element units,
// so that lanes reading granule i of consecutive units hit different banks without padding.
// The map is its own inverse.
__device__ __forceinline__ int swizzled_granule(int g) { return (g & ~15) | ((g & 15) ^ ((g >> 4) & 15)); }
struct SwizzledX {
    const uint8_t* xs;
    __device__ __forceinline__ float4 operator()(int col) const { return *(const float4*)(xs + 16 * swizzled_granule(col >> 2)); }
};

template <int FMT> struct SpanFmt;

template <> struct SpanFmt<QMOE_FMT_Q8_0> {
    static constexpr int PP4 = 17, MEM4 = 272;       // pieces and memory bytes per four units
    static constexpr bool LINEAR = true;             // piece t of the image is memory byte 16 t
    __device__ __forceinline__ static int src(int t) { return 16 * t; }
    // where in the image the reads of unit u start
    __device__ __forceinline__ static int unit_offset(int u) { return u * 68; }
    __device__ __forceinline__ static void read(const uint8_t* at, int, uint32_t* r) {
        const uint32_t* p = (const uint32_t*)at;
#pragma unroll
        for (int i = 0; i < 17; ++i) r[i] = p[i];
    }
};
template <> struct SpanFmt<QMOE_FMT_Q5_K> {
    static constexpr int PP4 = 11, MEM4 = 176;
    static constexpr bool LINEAR = true;
    __device__ __forceinline__ static int src(int t) { return 16 * t; }
    __device__ __forceinline__ static int unit_offset(int u) { return (u >> 2) * 176 + 8 * (u & 3); }
    __device__ __forceinline__ static void read(const uint8_t* at, int u, uint32_t* r) {   // at = block + 8 c
        const int c = u & 3;
        const uint4 hdr = *(const uint4*)(at - 8 * c);
        r[0] = hdr.x; r[1] = hdr.y; r[2] = hdr.z; r[3] = hdr.w;
        const uint2 qh = *(const uint2*)(at + 16);
        r[4] = qh.x; r[5] = qh.y;
#pragma unroll
        for (int g2 = 0; g2 < 4; ++g2) {
            const uint2 qs = *(const uint2*)(at + 48 + 32 * g2);
            r[6 + 2 * g2] = qs.x; r[7 + 2 * g2] = qs.y;
        }
    }
};
template <> struct SpanFmt<QMOE_FMT_Q4_K> {
    static constexpr int PP4 = 9, MEM4 = 144;
    static constexpr bool LINEAR = true;
    __device__ __forceinline__ static int src(int t) { return 16 * t; }
    __device__ __forceinline__ static int unit_offset(int u) { return (u >> 2) * 144 + 8 * (u & 3); }
    __device__ __forceinline__ static void read(const uint8_t* at, int u, uint32_t* r) {   // at = block + 8 c
        const int c = u & 3;
        const uint4 hdr = *(const uint4*)(at - 8 * c);
        r[0] = hdr.x; r[1] = hdr.y; r[2] = hdr.z; r[3] = hdr.w;
#pragma unroll
        for (int g2 = 0; g2 < 4; ++g2) {
            const uint2 qs = *(const uint2*)(at + 16 + 32 * g2);
            r[4 + 2 * g2] = qs.x; r[5 + 2 * g2] = qs.y;
        }
    }
};
template <> struct SpanFmt<QMOE_FMT_Q6_K> {
    static constexpr int PP4 = 14, MEM4 = 210;
    static constexpr bool LINEAR = false;
    __device__ __forceinline__ static int src(int t) {
        const int blk = t / 14, piece = t - 14 * blk;
        return blk * 210 + (piece < 13 ? 16 * piece : 194);
    }
    __device__ __forceinline__ static int unit_offset(int u) { return (u >> 2) * 224 + 64 * ((u >> 1) & 1) + 16 * (u & 1); }
    __device__ __forceinline__ static void read(const uint8_t* at, int u, uint32_t* r) {   // at = block + 64 h + 16 c
        const int h = (u >> 1) & 1, c = u & 1;
        const uint8_t* b = at - 64 * h - 16 * c;
        const uint4 la = *(const uint4*)at;
        const uint4 lb = *(const uint4*)(at + 32);
        const uint4 hq = *(const uint4*)(b + 128 + 32 * h + 16 * c);
        const uint2 sc = *(const uint2*)(b + 192 + 8 * h);
        r[0] = la.x; r[1] = la.y; r[2] = la.z; r[3] = la.w;
        r[4] = lb.x; r[5] = lb.y; r[6] = lb.z; r[7] = lb.w;
        r[8] = hq.x; r[9] = hq.y; r[10] = hq.z; r[11] = hq.w;
        const uint32_t s0 = sc.x >> (8 * c), s1 = sc.y >> (8 * c);
        r[12] = (s0 & 0xFFu) | ((s0 >> 8) & 0xFF00u);
        r[13] = (s1 & 0xFFu) | ((s1 >> 8) & 0xFF00u);
        r[14] = *(const uint16_t*)(b + 222);
    }
};

// A ring slot holds the image of 64 units.
template <int FMT> struct SpanSlot {
    static constexpr int BYTES = SpanFmt<FMT>::PP4 * 256;
    static constexpr int CHUNKS = (BYTES + 1023) / 1024;                     // load instructions of a whole slot
    static constexpr int LAST_LANES = (BYTES - (CHUNKS - 1) * 1024) / 16;    // lanes of the last one
};

// One problem of a launch, as the kernel sees it.
struct SpanProblem {
    const uint8_t* w;    // [n, k] packed rows
    const uint8_t* w2;   // second matrix of a gate/up pair, or null
    void* y;             // n outputs
    int n, k;
    int first_item, end_item;   // the problem's range of the launch's work items
    int ydt;
    int key;             // which activation row it reads
};
// One activation row: consecutive problems that read the same row share it.
struct SpanKey {
    const void* x;
    int k, xdt;
    int offset;          // where the row lies in the activation area of LDS (bytes)
    int pad;
};
struct SpanArgs {
    int count, keys, items, pad;
    uint32_t* status;     // the device's launch status word (a wave whose bounded wait expires raises it)
    int64_t wait_ticks;   // bound of a wait for the workgroup's other waves, in 100 MHz ticks; < 0: expire at once
    SpanProblem p[STREAM_MAX_PROBLEMS];
    SpanKey key[SPAN_MAX_KEYS];
};

bool span_supported(const StreamArgs& args);
int span_launch(const StreamArgs& args, hipStream_t s);

}  // namespace qmoe
