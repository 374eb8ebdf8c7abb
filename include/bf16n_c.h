/* C ABI of libbf16n_hip.so — the drop-in boundary of the BF16N hot path on MI355X (gfx950).
 *
 * Plain pointers and sizes only.  Every function returns a status: BF16N_OK, BF16N_EINVAL (the reference throws
 * std::invalid_argument with the same message) or BF16N_ERUNTIME (std::runtime_error: HIP errors, encoder invariants);
 * bf16n_last_error() gives the message of the calling thread's last failure.  `stream` is a hipStream_t passed as
 * void* (NULL = the default stream).  Launchers only enqueue kernels: no allocation, no host synchronisation, no
 * environment reads, so they can be captured into HIP graphs after bf16n_init().  All device pointers are the caller's.
 *
 * Each entry point names the reference interface it replaces (paths relative to the reference repository root).
 * The C++ API of the reference (namespace bf16n, core/include/bf16n/{encode,policy,launch}.h) is provided on top of
 * this file by the headers under include/bf16n/ with the same names, argument meaning and exceptions.
 */
#ifndef BF16N_C_H
#define BF16N_C_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { BF16N_OK = 0, BF16N_EINVAL = 1, BF16N_ERUNTIME = 2 };
enum { BF16N_FMT_NIBBLE = 1, BF16N_FMT_HUFFMAN = 2, BF16N_FMT_HUFPAIR = 3 };
enum { BF16N_FLAG_CHUNK_MAJOR = 1, BF16N_FLAG_FRAG_ORDER = 2, BF16N_FLAG_WAVE64 = 4 };
enum { BF16N_ENGINE_LLAMA = 0, BF16N_ENGINE_VLLM = 1, BF16N_ENGINE_MI355X = 2 };
enum { BF16N_MODE_HYBRID = 0, BF16N_MODE_HUFFMAN = 1, BF16N_MODE_NIBBLE = 2 };

const char * bf16n_last_error(void);
/* No counterpart in the reference.  The kernel instance that the calling thread's last dense product launch chose, in
 * the profiler's spelling ("k_w64_mmv<bf16_t, 4, 1, 2, 1>"), set by the dispatch code; "" where a path leaves no note.
 * For measurement programs that name the kernel they time.  Valid until the thread's next call of this function. */
const char * bf16n_last_kernel(void);

/* ---- host encoder: bf16n::encode, core/include/bf16n/encode.h:12-26, core/src/encode.cpp:443-526 ----------------- */
typedef struct bf16n_encoded bf16n_encoded; /* owns plane + aux (struct encoded, encode.h:12-17) */
/* w: rows x K BF16 bit patterns, row-major (host).  flags: BF16N_FLAG_* layout bits (chunk_major / frag_order arguments
 * of the reference; FRAG_ORDER is rejected with EINVAL, WAVE64 is this build's wave64 stream layout).  R: rows per unit,
 * {1, 2, 4, 8, 16} as in the reference, or 32 with WAVE64 for 32-row x 256-column tiles in matrix-core operand order. */
int bf16n_encode(const uint16_t * w, int64_t rows, int64_t K, int format, int R, uint32_t flags, bf16n_encoded ** out);
const uint8_t * bf16n_encoded_plane(const bf16n_encoded * e, uint64_t * bytes);
const uint8_t * bf16n_encoded_aux(const bf16n_encoded * e, uint64_t * bytes);
int  bf16n_encoded_format(const bf16n_encoded * e); /* format actually produced (HUFPAIR may fall back to HUFFMAN) */
int  bf16n_encoded_R(const bf16n_encoded * e);      /* rows per unit, 0 for NIBBLE */
void bf16n_encoded_free(bf16n_encoded * e);
/* worker threads of the encoder (the reference fixes min(12, cores), encode.cpp:27); 0 = default min(16, cores) */
void bf16n_set_encode_threads(int n);

/* ---- shape policy: bf16n::choose, core/include/bf16n/policy.h:12-38, core/src/policy.cpp:45-69 -------------------- */
/* out[5] = {format, R, chunk_major, frag_order, wave64}.  Returns 1 if a choice was made, 0 if the shape stays BF16
 * (std::nullopt).  Never fails.  engine MI355X: the reference's llama rules with unit sizes chosen for 256 CUs of
 * wave64 and the wave64 stream layout where the shape allows it; experts with a multiple of 32 rows get R = 32 tiles,
 * and so do, with dense_frag_order set, dense matrices of at least 131072 rows (a multiple of 32), K >= 1024. */
int bf16n_choose(int64_t rows, int64_t K, int64_t n_matrices, int engine, int mode, int64_t dense_min, int expert,
                 int dense_frag_order, int * out);

/* ---- device view of one encoded matrix: struct weight, core/include/bf16n/launch.h:15-25 --------------------------- */
typedef struct bf16n_weight {
    const uint8_t * plane; /* device, 16-byte aligned */
    const uint8_t * aux;   /* device, 16-byte aligned */
    int32_t  format, R;
    int64_t  K, rows;
    uint32_t flags;        /* BF16N_FLAG_* from the aux header (cm / fo booleans of the reference) */
    uint32_t pad_;
    uint64_t off_a, off_b, off_c, off_d;
} bf16n_weight;

/* struct mmv_args, core/include/bf16n/launch.h:27-44: same fields and meaning (signed strides in bytes) */
typedef struct bf16n_mmv_args {
    const void * x; void * y; const void * ids;
    int64_t x_tok, y_tok, ids_s0, ids_s1, x_slot, y_slot;
    int64_t rows_per_matrix, row0, nrows;
    int32_t ncols, n_used, x_per_slot;
    uint8_t x_bf16, y_bf16, pad_[2];
} bf16n_mmv_args;

/* ---- launchers: core/include/bf16n/launch.h:46-83, core/src/launch.cu ------------------------------------------------ */
int bf16n_init(void);                 /* init(), launch.h:47, launch.cu:270-306: once per process, before graph capture */
int bf16n_cu_count(int * out);        /* sm_count(), launch.h:48 */
int bf16n_mmv(const bf16n_weight * w, const bf16n_mmv_args * a, void * stream, int multi_col); /* mmv, launch.h:52, launch.cu:313-325 */
/* (multi_col, launch.h:52: columns of a dense batch may share decodes.  0: every column has the bits of its own
 * single-column launch.  Non-zero: the same, except where a dense batch of BF16 columns runs on the matrix cores (tile
 * layout; the 4-bit code from two columns on for matrices that fill the GPU): there a column has the same bits at every
 * batch size and position, another summation order than the single-column GEMV, the same error bound.) */
/* the dense dispatch rule: BF16 token columns up to which bf16n_mmv beats dequant + GEMM for this matrix (8, the
 * reference's fixed rule, core/torch/torch_bindings.cpp:195 and ops.py:25-27; 16 for matrices of 128 Mi weights and more
 * in wave64 units; 64 for the 4-bit code where its batches run on the matrix cores at every count, 16 where up to 16
 * columns; 512 for tile-layout matrices there) */
int bf16n_gemv_max_tokens(const bf16n_weight * w, int * out);
/* The dense path beyond bf16n_gemv_max_tokens: y (n_tok x rows, BF16) = x (n_tok x K, BF16) W^T through exact dequant of
 * the matrix, in pieces of at most 64 MiB, into `scratch`, and a stock BF16 GEMM with FP32 accumulation (hipBLASLt) on
 * each piece: what the reference's llama.cpp adapter does above 8 tokens with a pool allocation and cuBLAS
 * (engines/llamacpp/patches/0002-...patch:423-437, switch at :157) and its torch binding with at::mm
 * (core/torch/torch_bindings.cpp:195-239).  Row strides in elements.  Nothing is allocated in the call: scratch (at
 * least one unit of decoded rows; *scratch_bytes of bf16n_linear_dense_sizes for the fewest pieces) and the GEMM
 * workspace (*gemm_workspace_bytes) are the caller's.  Call bf16n_linear_dense_sizes once before capturing the call
 * into a HIP graph: it loads the BLAS and creates its handle. */
int bf16n_linear_dense_sizes(const bf16n_weight * w, uint64_t * scratch_bytes, uint64_t * gemm_workspace_bytes);
int bf16n_linear_dense(const bf16n_weight * w, const uint16_t * x, int64_t x_row, int n_tok, uint16_t * y, int64_t y_row,
                       void * scratch, uint64_t scratch_bytes, void * gemm_workspace, uint64_t gemm_workspace_bytes, void * stream);
int bf16n_mmv_glu(const bf16n_weight * w, const bf16n_mmv_args * a, void * stream);            /* mmv_glu merged [gate;up], launch.h:55, launch.cu:327-339 */
int bf16n_mmv_glu2(const bf16n_weight * gate, const bf16n_weight * up, const bf16n_mmv_args * a, void * stream); /* mmv_glu(gate, up), launch.h:61, launch.cu:341-365 */
/* No counterpart in the reference (its engines run the router's softmax + top-k as a launch of their own between the
 * router's product and the experts').  bf16n_mmv_glu2 over routed experts that selects them in its own prologue: one
 * dependent launch fewer in a decode step.  a->ids: int32 id rows [tokens, n_used]; columns 0..k-1 are WRITTEN (the k
 * largest of softmax(logits row), ties to the lower index, as bf16n_router_topk_strided writes them), columns from k on
 * are read (experts every token uses).  weights: k softmax weights per token (renormalised to sum 1 if renorm) at
 * weights + token * weights_stride.  Expert stacks in the tile layout, BF16 activations, at most 256 experts. */
int bf16n_mmv_glu2_topk(const bf16n_weight * gate, const bf16n_weight * up, const bf16n_mmv_args * a, const float * logits,
                        int64_t logits_stride, int n_experts, int k, int renorm, float * weights, int64_t weights_stride, void * stream);
int bf16n_dequant(const bf16n_weight * w, int64_t row0, int64_t nrows, uint16_t * out, void * stream); /* dequant, launch.h:63, launch.cu:367-402 */
int bf16n_get_rows(const bf16n_weight * w, const void * ids, int64_t ids_s0, int64_t n, void * dst, int dst_bf16,
                   int64_t dst_s1, void * stream, int64_t row0);                                /* get_rows, launch.h:68-69, launch.cu:404-443 */
int bf16n_mm_ids_supported(const bf16n_weight * w, const bf16n_weight * up);                    /* launch.h:74, launch.cu:446-456; 1/0 */
int bf16n_mm_ids_route(const void * ids, int ids_i64, int64_t ids_row_stride, int32_t * ids_src1, int32_t * ids_dst,
                       int32_t * bounds, int n_experts, int n_tok, int n_used, int nchannels_y, int sis1, void * stream); /* launch.h:75-76, launch.cu:458-471, mmid_helper.cu */
int bf16n_mm_ids(const bf16n_weight * w, const bf16n_weight * up, const void * x_bf16, int64_t x_row,
                 const int32_t * ids_src1, const int32_t * ids_dst, const int32_t * bounds, void * dst, int dst_bf16,
                 int64_t dst_col, int n_experts, int n_tok, int n_used, void * stream);          /* launch.h:77-79, launch.cu:473-535 */
/* No counterpart in the reference.  bf16n_mm_ids for calls with many tokens per expert (prefill), in two phases through
 * a scratch buffer of the caller's: groups of experts are decoded once into the scratch (BF16, matrix-core operand
 * order) by a kernel with the GEMV's decode rate and multiplied from there by a kernel without a decoder; the fused
 * kernel of bf16n_mm_ids decodes an expert once per pass of 128 of its tokens.  Tile layout only.  scratch: 16-byte
 * aligned device memory of at least *per_expert bytes (bf16n_mm_ids_scratch_bytes; *advised is the size whose groups
 * stay in the last-level cache between the two kernels).  Same arguments and results as bf16n_mm_ids otherwise. */
int bf16n_mm_ids_scratch_bytes(const bf16n_weight * w, const bf16n_weight * up, int n_experts, uint64_t * per_expert, uint64_t * advised);
int bf16n_mm_ids_scratch(const bf16n_weight * w, const bf16n_weight * up, const void * x_bf16, int64_t x_row,
                         const int32_t * ids_src1, const int32_t * ids_dst, const int32_t * bounds, void * dst, int dst_bf16,
                         int64_t dst_col, int n_experts, void * scratch, uint64_t scratch_bytes, void * stream);
/* No counterpart in the reference.  bf16n_mm_ids_route + bf16n_mm_ids in one call that allocates nothing, for callers
 * that cannot allocate device memory (code under HIP graph capture, tight serving loops, harnesses that forbid it): the
 * routing lists are kept in a device array that belongs to the library (about 516 KiB per GPU, held until the process
 * ends) instead of buffers of the caller.  ids: n_tok x n_used expert ids (int32, or int64 with ids_i64; row stride in
 * elements); per_slot: x holds one activation row per (token, slot) (the down product) instead of one per token.  At
 * most 65536 routed pairs (n_tok * n_used) and 1024 experts per call, EINVAL beyond.  dst gets the bits that
 * bf16n_mm_ids writes for the same arguments.  All calls on one GPU share the array: calls that can overlap on one GPU
 * (different streams, different threads) race; calls on one stream are ordered.  The ids of a token must name distinct
 * experts: a repeated naming is counted in the bounds but listed once (as in bf16n_mm_ids_route, mmid_helper.cu:66-71),
 * and the list entry it leaves unwritten is whatever an earlier call left in the array.  Call bf16n_init() on every GPU
 * before the first capture. */
int bf16n_moe_mm_ids_static(const bf16n_weight * w, const bf16n_weight * up, const void * x_bf16, int64_t x_row, const void * ids,
                            int ids_i64, int64_t ids_row_stride, int per_slot, void * dst, int dst_bf16, int64_t dst_col,
                            int n_experts, int n_tok, int n_used, void * stream);
int bf16n_moe_combine(const float * ys, const void * w, int w_bf16, void * y, int y_bf16, int n_tok, int n_used,
                      int64_t n, void * stream);                                                /* launch.h:82-83, launch.cu:562-572 */
int bf16n_swiglu(const float * g, const float * u, float * y, int64_t n, void * stream);       /* launch.h:85, launch.cu:574-582 */
/* Engine glue of a decode step in one launch (the reference leaves it to the engines): per token, in FP32,
 *   sum = a + b + c + sum_k wts[k] * ys[k]     (BF16 rows a, b, c of n elements; FP32 rows ys of n_used slots, combined
 *                                                by bf16n_moe_combine's fmaf chain; every addend but a may be null)
 *   y_sum = bf16(sum) if non-null;  y_norm = bf16(sum * rsqrt(mean(sum^2) + eps) * gamma)  (gamma: n BF16 values or null) */
int bf16n_add_rmsnorm(const uint16_t * a, const uint16_t * b, const uint16_t * c, const float * ys, const void * wts, int wts_bf16,
                      int n_used, const uint16_t * gamma, uint16_t * y_sum, uint16_t * y_norm, int n_tok, int64_t n, float eps,
                      void * stream);

/* Router softmax + top-k on the device, so that a whole MoE decode step can be captured into one HIP graph.  The
 * reference leaves this to the engines (vllm_bf16n/moe.py:62-67 receives topk_weights/topk_ids); it has no core
 * counterpart.  logits: n_tok x n_experts FP32 (row stride in elements); ids: n_tok x k int32; weights: n_tok x k FP32,
 * softmax probabilities of the k largest logits (ties: lower index), renormalised to sum 1 when renorm != 0. */
int bf16n_router_topk(const float * logits, int64_t logits_stride, int n_tok, int n_experts, int k, int renorm,
                      int32_t * ids, float * weights, void * stream);
/* the same into rows of out_stride >= k elements: a caller that always runs further experts beside the routed ones (a
 * shared expert stacked behind them) keeps their ids and weights in the columns from k on */
int bf16n_router_topk_strided(const float * logits, int64_t logits_stride, int n_tok, int n_experts, int k, int renorm,
                              int32_t * ids, float * weights, int64_t out_stride, void * stream);
/* bf16n_router_topk_strided and bf16n_mm_ids_route (launch.cu:458-471) in one launch for few tokens: after the top-k the
 * same block sorts the first n_slots columns (k <= n_slots <= out_stride: the k chosen here, then the columns the caller
 * keeps filled) of the id rows into the lists bf16n_mm_ids_route writes for them, over n_listed >= n_experts experts
 * (bounds: n_listed + 1 entries; ids_src1, ids_dst: n_tok * n_slots).  Limits, bf16n_router_topk_route_fits: n_tok <= 16,
 * n_tok * n_slots <= 1024, n_listed <= 1024.  Ids outside [0, n_listed) in the caller's columns are left out of the lists. */
int bf16n_router_topk_route_fits(int n_tok, int n_slots, int n_listed);
int bf16n_router_topk_route(const float * logits, int64_t logits_stride, int n_tok, int n_experts, int k, int renorm,
                            int32_t * ids, float * weights, int64_t out_stride, int n_slots, int n_listed,
                            int32_t * ids_src1, int32_t * ids_dst, int32_t * bounds, int nchannels_y, int sis1, void * stream);

/* ---- load-time conversion and the registry of resident tensors: the reference's llama.cpp adapter without ggml types
 * (engines/llamacpp/patches/0002-ggml-cuda-thin-BF16N-adapter-over-the-shared-core.patch).  An engine stores a converted
 * tensor as rows * K bytes of device memory (the plane); the aux buffer is allocated here and found again by the
 * address of the tensor's data.  These calls allocate and synchronise: load time only, never under graph capture. ---- */
/* ggml_backend_cuda_bf16n_choose, patch 0002:258-268: 0 = stay BF16, 1 = NIBBLE, 2 = Huffman family.  Never fails. */
int bf16n_adapter_choose(int64_t rows, int64_t K, int64_t n_matrices, const char * mode, int64_t dense_min, int expert, int engine);
/* ggml_backend_cuda_bf16n_convert, patch 0002:271-329: encode the host BF16 tensor (n_matrices x rows_per_matrix x K)
 * with the layout the engine's policy picks for format_tag (1 NIBBLE, 2 Huffman family; matrix_core_order: the policy's
 * dense_frag_order), copy the plane into tensor_data (device, rows * K bytes, 16-byte aligned), allocate and fill the
 * aux buffer, register the tensor under `owner`, decode it on the device and compare every weight with the source.
 * *roundtrip_ok = 1 when they are identical; verbose: one line per tensor on stderr as the reference prints. */
int bf16n_adapter_convert(void * tensor_data, const void * bf16_host, int64_t rows_per_matrix, int64_t K, int64_t n_matrices,
                          int format_tag, int engine, int matrix_core_order, const void * owner, const char * name, int verbose,
                          int * roundtrip_ok);
/* the verify step alone (patch 0002:309-322; roundtrip_equal of vllm_bf16n/ops.py): device decode against a host source */
int bf16n_verify_roundtrip(const bf16n_weight * w, const uint16_t * bf16_host, int * ok);
/* a tensor the caller encoded and uploaded itself joins the registry (its aux buffer stays the caller's) */
int bf16n_adapter_register(const bf16n_weight * w, const void * owner);
/* lookup, patch 0002:73-92: the registered tensor whose plane holds address p (any row start: views of whole rows);
 * *found = 0 if none.  The weight is returned by value. */
int bf16n_adapter_lookup(const void * p, bf16n_weight * out, int64_t * row0, int * found);
/* ggml_cuda_bf16n_free, patch 0002:121-132: drop every tensor of `owner` (before its buffer is freed); *n: how many */
int bf16n_adapter_release(const void * owner, int * n);
int bf16n_adapter_count(void);

#ifdef __cplusplus
}
#endif
#endif
