// Decoder of the wave64 HUFPAIR layout (FLAG_WAVE64), shared by the GEMV / dequant kernels and the batched MoE kernel.
#pragma once

#include "bf16n_c.h"
#include "dev_common.h"

namespace bf16n {
namespace dev {

constexpr int RING = 512;     // ring words per wave (2 KiB)
constexpr int RING_PAD = 256; // copy of the first ring words behind the end: reads never wrap
constexpr int BLK = 256;      // words per refill block: one uint4 per lane
constexpr int AHEAD = 256;    // words kept ahead of the consumer: a unit start (192) or a step (4 x 64)
constexpr int LUT_WORDS = 1 << HP_LP;
constexpr int WAVE_LDS_WORDS = RING + RING_PAD;

// 16 bytes that a launch reads once, loaded with the non-temporal hint: 8 % faster on the 248320 x 2048 GEMV (126
// against 136 us). Planes that other columns or passes of the launch read again (routed experts with many tokens, small
// matrices in a column loop) keep the default policy, which is faster there. Stream blocks start on 128-byte lines, so
// no line belongs to two blocks (with the hint a shared line is fetched twice): the GEMVs and the routed batched
// kernels are faster with the hint inside a decode step, a large dense matrix in the batched tile kernel is not, so the
// stream hint is a flag of its own (w64_dec::once)
typedef uint32_t u32x4_nt __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_once(const uint4 * p) {
    const u32x4_nt v = __builtin_nontemporal_load((const u32x4_nt *) p);
    return make_uint4(v.x, v.y, v.z, v.w);
}

// A byte range of device memory behind a buffer descriptor.  The decode loops prefetch a fixed distance ahead with
// loads that are issued unconditionally (so that the count of loads in flight at every wait is known at compile time);
// near the end of a wavefront's range those loads point past it.  Through a descriptor such a load is dropped by the
// address unit and returns zeros: no memory request (clamping the address to the last block instead re-fetched it, and
// with the non-temporal hint every such repeat went to memory again: 3 KiB per decode chain, 3.6 % of the traffic of
// the output projection).  The whole offset travels in the vector operand, which is what the range check looks at.
typedef __amdgpu_buffer_rsrc_t range_t;
__device__ __forceinline__ range_t make_range(const void * base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int) bytes, 0x00020000); // raw buffer, 32-bit data
}
template <bool ONCE>
__device__ __forceinline__ uint4 range_load16(range_t r, uint32_t byte_off) {
    const u32x4_nt v = ONCE ? __builtin_amdgcn_raw_buffer_load_b128(r, (int) byte_off, 0, 2)   // nt
                            : __builtin_amdgcn_raw_buffer_load_b128(r, (int) byte_off, 0, 0);
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint4 range_load16(range_t r, uint32_t byte_off, bool once) {
    return once ? range_load16<true>(r, byte_off) : range_load16<false>(r, byte_off);
}

struct w64_ptrs { const uint8_t * plane; const uint32_t * lut; const uint32_t * ubase; const uint32_t * stream; };
__device__ __forceinline__ w64_ptrs w64p(const bf16n_weight & w) {
    return {w.plane, (const uint32_t *) (w.aux + w.off_a), (const uint32_t *) (w.aux + w.off_b), (const uint32_t *) (w.aux + w.off_d)};
}

__device__ __forceinline__ uint32_t lds_entry(const uint32_t * lut, uint32_t byte_off) {
    return *(const uint32_t *) ((const char *) lut + byte_off);
}
__device__ __forceinline__ uint32_t uniform(uint32_t v) { return (uint32_t) __builtin_amdgcn_readfirstlane((int) v); }
// lane mask of (a < b), unsigned: one v_cmp into a scalar register pair, used both as the vote and as the select mask
// (written out because the compiler otherwise materialises the same comparison twice, once per use)
__device__ __forceinline__ uint64_t lanes_lt(uint32_t a, uint32_t b) {
    uint64_t m;
    asm("v_cmp_lt_u32_e64 %0, %1, %2" : "=s"(m) : "v"(a), "v"(b));
    return m;
}
// lane mask of (a != b)
__device__ __forceinline__ uint64_t lanes_ne(uint32_t a, uint32_t b) {
    uint64_t m;
    asm("v_cmp_ne_u32_e64 %0, %1, %2" : "=s"(m) : "v"(a), "v"(b));
    return m;
}
// lane-wise m ? b : a
__device__ __forceinline__ uint32_t pick(uint32_t a, uint32_t b, uint64_t m) {
    uint32_t d;
    asm("v_cndmask_b32_e64 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "s"(m));
    return d;
}
__device__ __forceinline__ int64_t uniform64(int64_t v) { // an offset the compiler may keep in scalar registers
    return (int64_t) (((uint64_t) uniform((uint32_t) ((uint64_t) v >> 32)) << 32) | uniform((uint32_t) v));
}

// Decoder state of one wave.  cons / filled / limit are the same in every lane (scalar registers).
// HINT: the load policy of the stream blocks, -1 a run-time flag (`once`), 0 plain, 1 non-temporal.  As a compile-time
// choice it keeps the loads of a decode loop out of branches (a loop with the two load forms side by side moved every
// prefetched block between registers at its end: 2.5 % of the 248320 x 2048 GEMV).
template <int HINT = -1>
struct w64_dec_t {
    uint32_t w0, w1, w2;    // per lane: three stream words
    uint32_t P;             // per lane: bits consumed since the unit began, in its low seven bits (the bits above are
                            // scraps of table entries); P mod 32 is the position in w0, which is all the funnel shift reads
    uint32_t P5;            // bit 5 of P at the last check: a change of that bit is a word boundary passed
    uint32_t nw;            // the word requested at the last check (becomes w2 where took is set)
    uint64_t took;          // lanes that requested a word at the last check
    uint32_t cons;          // words consumed, relative to src
    uint32_t filled;        // words copied into the ring, relative to src (multiple of BLK)
    uint32_t * ring;
    range_t src;            // the blocks that hold words of this wave (starts on a 128-byte line)
    uint4 pend;             // the block that starts at `filled`, in flight
    uint4 first_blk;        // the first block between start and start_finish
    int lane;
    bool once;              // stream blocks with the non-temporal hint (same in every lane)

    // Every load is unconditional (a block past the end is dropped by the range check and reads as zeros) so that the
    // number of loads in flight at any point of the loop is fixed and the waits for prefetched data never drain newer
    // loads.
    __device__ __forceinline__ uint4 load_block(uint32_t first_word) const {
        if constexpr (HINT < 0) {
            return range_load16(src, 4 * first_word + 16 * (uint32_t) lane, once);
        } else {
            return range_load16<HINT == 1>(src, 4 * first_word + 16 * (uint32_t) lane);
        }
    }
    __device__ __forceinline__ void store_block(uint32_t first_word, const uint4 v) {
        const uint32_t off = first_word & (RING - 1);
        *((uint4 *) (ring + off) + lane) = v;
        if (off == 0) {
            *((uint4 *) (ring + RING) + lane) = v;
        }
    }
    // stream words [first, end) of the aux stream belong to this wave
    __device__ __forceinline__ void start(uint32_t * ring_, const uint32_t * stream, uint32_t first, uint32_t end, int lane_, bool once_ = false,
                                          bool split = false) {
        ring = ring_;
        lane = lane_;
        once = once_;
        // blocks start on 128-byte lines (a block is then eight whole cache lines, and no line belongs to two blocks):
        // up to 31 words before `first`, which are skipped; before the first unit of a matrix these are the last words
        // of the section that precedes the stream in the same buffer (the header and the table come first)
        const uint32_t a4 = first & ~3u;
        const int32_t a = (int32_t) a4 - (int32_t) (((uintptr_t) (stream + a4) & 127u) >> 2);
        cons = (uint32_t) ((int32_t) first - a);
        // whole blocks up to the one that holds the last word (the stream is padded: a block may run past `end`)
        const uint32_t blocks = (uint32_t) ((int32_t) end - a - 1) / BLK + 1;
        src = make_range(stream + (int32_t) uniform((uint32_t) a), uniform(blocks * BLK * 4));
        first_blk = load_block(0);
        pend = load_block(BLK);
        if (!split) {
            start_finish();
        }
    }
    // the second half of start(..., split = true): callers put other loads between the request of a chain's first
    // blocks and the wait for them
    __device__ __forceinline__ void start_finish() {
        store_block(0, first_blk);
        filled = BLK;
    }
    // at least AHEAD words in the ring beyond the consumer; the block after them in flight.  At most one block per
    // call is the steady state (a step consumes 85 words on average, 256 at most); the loop only runs when a wave
    // starts.  The next block is requested only when the one in flight has been stored: one load per ring slot.
    __device__ __forceinline__ void keep_ahead() {
        if (filled - cons < AHEAD) {
            store_block(filled, pend);
            filled += BLK;
            while (filled - cons < AHEAD) {
                store_block(filled, load_block(filled));
                filled += BLK;
            }
            pend = load_block(filled);
        }
    }
    __device__ __forceinline__ void begin_unit() {
        const uint32_t * p = ring + (cons & (RING - 1)) + 3 * lane;
        w0 = p[0];
        w1 = p[1];
        w2 = p[2];
        P = 0;
        P5 = 0;
        took = 0;
        nw = 0;
        cons = uniform(cons + 192);
    }
    // two pair codes; afterwards lanes whose position passed a word boundary request the next stream words in lane order
    __device__ __forceinline__ void two(const uint32_t * lut, uint32_t & e0, uint32_t & e1) {
        two_with([lut](uint32_t off) { return lds_entry(lut, off); }, e0, e1);
    }
    // the same with the table at LDS byte address `lut_addr`, a compile-time value at the call (kernels whose only LDS
    // is the dynamic segment keep their tables at its start, address 0): the address of an entry is then the masked
    // stream bits themselves plus an immediate, where a pointer into the dynamic segment costs an add per lookup
    __device__ __forceinline__ void two_at(uint32_t lut_addr, uint32_t & e0, uint32_t & e1) {
        two_with([lut_addr](uint32_t off) {
            return *(const __attribute__((address_space(3))) uint32_t *) (uintptr_t) (lut_addr + off);
        }, e0, e1);
    }
    template <typename L>
    __device__ __forceinline__ void two_with(L entry, uint32_t & e0, uint32_t & e1) {
        const uint32_t W = __builtin_amdgcn_alignbit(w1, w0, P);
        e0 = entry(W & 0x3FFCu);
        const uint32_t W2 = W >> (e0 & 31u);
        e1 = entry(W2 & 0x3FFCu);
        // entry bits 5 and 6 are zero: the low seven bits of the running sum are exact (the exponent fields only add
        // above them), and two pair codes are at most 24 bits, so bit 5 changes exactly when a word boundary is passed
        P = P + e0 + e1;
        const uint32_t p5 = P & 32u;
        const uint64_t m = lanes_ne(p5, P5);
        P5 = p5;
        const uint32_t rank = __builtin_amdgcn_mbcnt_hi((uint32_t) (m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t) m, 0u));
        const uint32_t req = ring[(cons & (RING - 1)) + rank];
        // the word requested one check ago has arrived by now: it is this lane's w2
        w2 = pick(w2, nw, took);
        w0 = pick(w0, w1, m);
        w1 = pick(w1, w2, m);
        nw = req;
        took = m;
        cons = uniform(cons + (uint32_t) __builtin_popcountll(m));
    }
    // the 16 weights of this lane in one step as 8 BF16 pairs: wp[2j], wp[2j+1] = columns 128j + 4(lane%32) + {0,1}, {2,3}
    __device__ __forceinline__ void step(const uint32_t * lut, const uint4 sm, uint32_t (&wp)[8]) {
        const uint32_t smw[4] = {sm.x, sm.y, sm.z, sm.w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            uint32_t e0, e1;
            two(lut, e0, e1);
            wp[2 * j] = merge(spread_lo(smw[j]), e0);
            wp[2 * j + 1] = merge(spread_hi(smw[j]), e1);
        }
    }
};
typedef w64_dec_t<-1> w64_dec;

// Every block of a launch stages the same 16 KiB; the blocks start at different 1 KiB pieces of it so that they do not
// all ask for the same cache lines at the same moment.
__device__ __forceinline__ void stage_lut(uint32_t * lut, const uint32_t * lut_g) {
    const int rot = (int) ((blockIdx.x + 5 * blockIdx.y) * 64) & (LUT_WORDS / 4 - 1);
    for (int i = threadIdx.x; i < LUT_WORDS / 4; i += blockDim.x) {
        const int k = (i + rot) & (LUT_WORDS / 4 - 1);
        ((uint4 *) lut)[k] = ((const uint4 *) lut_g)[k];
    }
}

} // namespace dev
} // namespace bf16n
