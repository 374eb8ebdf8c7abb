/* TEST INFRASTRUCTURE ONLY — CPU restatement of the BF16N algorithms (plain C99).
 *
 * Nothing in the shipped library links, imports or calls this file; it exists so that tests, the smoke check and the
 * benchmark's cpu_baseline leg have an independent checker for the HIP path.
 *
 * Each function names the reference file:line it follows (paths relative to the reference repository root).
 *
 * Pinning status (what each function has been checked against, see tests/test_oracle_*.py):
 *   orc_plane, orc_encode (NIBBLE, HUFFMAN, HUFPAIR row-/chunk-major, fallback)   byte-for-byte against the reference
 *       encoder compiled from its own sources (oracle/_ref) and against committed golden fixtures made by it;
 *       Huffman code lengths additionally against a brute-force optimal length-limited code on tiny alphabets, Kraft
 *       equality and cost equality.  Where several symbols share a frequency the reference's tie order comes from an
 *       unstable std::sort; this file breaks ties by symbol value, so aux bytes can differ from the reference's in such
 *       a case while cost, Kraft sum and decoded weights never do (tests state which comparison they use).
 *   orc_decode   against the reference encoder's output (decode(encode(w)) == w for every format/layout, special BF16
 *       classes included) and the golden fixtures.
 *   orc_decode_w64 (this build's layout, no reference counterpart)   decode(encode(w)) == w, equality with orc_decode of
 *       the reference layout of the same tensor, and — for the R = 32 tile form — the tile mapping restated in numpy from
 *       its definition (tests/test_encoder_host.py: the permuted matrix encodes to the same plane and stream; a lane's 16
 *       weights of a step are two runs of 8 consecutive columns of one row).
 *   orc_gemv_*   against numpy float64 on exact weights (bound 1e-5 * sum|w x|) and one-hot known answers.
 *   orc_route    against a brute-force stable sort of (expert, token) pairs.
 *   orc_router_topk   no counterpart in the reference core (engine op): pinned by closed forms only (softmax sums to 1,
 *       ordering, ties to the lower index) — "parity unpinned" with respect to the reference.
 */
#ifndef BF16N_ORACLE_H
#define BF16N_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ORC_FMT_NIBBLE = 1, ORC_FMT_HUFFMAN = 2, ORC_FMT_HUFPAIR = 3 };
enum { ORC_FLAG_CHUNK_MAJOR = 1, ORC_FLAG_WAVE64 = 4 };

/* core/include/bf16n/format.h:41-47 — first 80 bytes of every aux buffer */
typedef struct {
    uint32_t magic, format, K, R;
    uint64_t rows;
    uint64_t off_a, off_b, off_c, off_d;
    uint64_t n_a, n_b;
    uint32_t flags, pad_;
} orc_header;

/* column inside a 512-chunk of slot s (0..15) of lane l (0..31); core/include/bf16n/format.h:51 */
int orc_pos_of(int l, int s);

/* sign|mantissa plane, row-major units; core/src/encode.cpp:48-62 */
void orc_plane(const uint16_t *w, int64_t rows, int64_t K, uint8_t *plane);

/* Length-limited Huffman code lengths by package-merge; core/src/encode.cpp:182-218.
 * freq[n] (zero = unused symbol), len[n] out.  Ties between equal frequencies: lower symbol first. */
void orc_limited_lengths(const uint64_t *freq, int n, int L, int *len);

/* Full encoder; core/src/encode.cpp:443-526 (argument contract :445-473).
 * plane: rows*K bytes (caller).  *aux is malloc'ed (free with orc_free).  Returns 0, or -1 for a contract violation
 * (message in orc_last_error()).  format_out: format actually produced (HUFPAIR may fall back to HUFFMAN). */
int orc_encode(const uint16_t *w, int64_t rows, int64_t K, int format, int R, int chunk_major, uint8_t *plane,
               uint8_t **aux, uint64_t *aux_bytes, int *format_out);
void orc_free(void *p);
const char *orc_last_error(void);

/* Independent decoder written from the layout alone; core/tests/test_encode.cpp:87-164.
 * Returns 0 or -1 (bad header). out: rows*K BF16 bit patterns, row-major. */
int orc_decode(const uint8_t *plane, const uint8_t *aux, uint64_t aux_bytes, uint16_t *out);

/* Decode of the wave64 layout (flag bit 2) that this build adds next to the reference layouts: same code, same LUT
 * semantics, 64 lanes per unit, one interleaved word stream per unit.  No reference counterpart: pinned only by
 * decode(encode(w)) == w and by comparing with orc_decode of the reference layout of the same tensor. */
int orc_decode_w64(const uint8_t *plane, const uint8_t *aux, uint64_t aux_bytes, uint16_t *out);
/* R = 32 tiles of the wave64 layout: index into the row-major rows x K matrix of element (vrow, vcol) of the 512-column
 * matrix the tile units are stored as. */
int64_t orc_tile32_index(int64_t vrow, int64_t vcol, int64_t K);

/* y[r] = sum_k W[r,k] x[k] with FP32 fmaf in the summation order of the reference GEMV kernels:
 * lane accumulators a0..a3 over (chunk, j), (a0+a1)+(a2+a3), then a 32-lane xor butterfly
 * (core/include/bf16n/kernels.cuh:498-535, :119-125).  chunk_major != 0: per-chunk partial sums added per row
 * (kernels.cuh:944-986).  w: exact BF16 bits, row-major; x: FP32 (BF16 activations widened by the caller). */
void orc_gemv_f32(const uint16_t *w, int64_t rows, int64_t K, const float *x, int chunk_major, float *y);
/* FP64 reference and the bound scale S[r] = sum_k |w x|; tests/conftest.py:46-55 */
void orc_gemv_f64(const uint16_t *w, int64_t rows, int64_t K, const float *x, double *y, double *s);

/* Decode + GEMV straight from the encoded buffers (the path the GPU kernels fuse), rows [row0, row0+nrows), FP32 in the
 * order of orc_gemv_f32; NIBBLE adds escape products after the dense sum (kernels.cuh:178-186).  threads <= 1: scalar.
 * Returns 0 or -1. This is what bench.py times as the CPU baseline. */
int orc_decode_gemv(const uint8_t *plane, const uint8_t *aux, uint64_t aux_bytes, int64_t row0, int64_t nrows,
                    const float *x, float *y, int threads);

/* silu(g) * u with silu(x) = x / (1 + expf(-x)); core/src/launch.cu:554-558, compat.cuh:31 */
void orc_swiglu(const float *g, const float *u, float *y, int64_t n);
/* y[t,i] = sum_k w[t,k] * ys[t,k,i] in slot order with fmaf; core/src/launch.cu:539-552 */
void orc_moe_combine(const float *ys, const float *w, float *y, int n_tok, int n_used, int64_t n);
/* Routing lists sorted by expert then token; core/src/mmid_helper.cu:48-136.
 * ids[t*ids_stride + k]; ids_src1[j] = t*sis1 + k % nchannels_y; ids_dst[j] = t*n_used + k; bounds[n_experts+1]. */
void orc_route(const int32_t *ids, int64_t ids_stride, int n_experts, int n_tok, int n_used, int nchannels_y, int sis1,
               int32_t *ids_src1, int32_t *ids_dst, int32_t *bounds);
/* softmax over n logits (FP32, max-subtracted), the k largest probabilities (ties: lower index), renormalised to sum 1.
 * Not part of the reference core (the engines' own op). */
void orc_router_topk(const float *logits, int n, int k, int32_t *ids, float *weights);

#ifdef __cplusplus
}
#endif
#endif
