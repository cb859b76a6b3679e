/*
 * bhi.h -- C ABI of libbhi_hip.so: fused entropy-decode + GEMV for compressed BF16
 * weights on gfx950 (MI355X).
 *
 * Each entry point stands in for one torch custom op of the reference
 * (namespace "bf16_huffman_infer", schemas at
 * bf16_huffman_infer/src/bf16_huffman_infer.cpp:29-35, CUDA implementations
 * registered at bf16_huffman_infer/src/kernel.cu:922-930).  The arguments are the
 * op's tensors as raw device pointers, in the op's order, followed by the
 * dimensions the reference reads from tensor sizes and the HIP stream the reference
 * takes from torch (kernel.cu:30-38).
 *
 * Rules for every function:
 *   - all pointers are device pointers valid on the current HIP device;
 *   - the call only enqueues work on `stream` (a hipStream_t, NULL = default
 *     stream); it never synchronises, allocates, frees or keeps a pointer;
 *   - the return value is 0 on success, a negative BHI_E* code for a rejected
 *     argument, or a positive hipError_t from the launch; bhi_last_error_string()
 *     describes the last failure on the calling thread.
 */
#ifndef BHI_H
#define BHI_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BHI_EINVAL   (-1)   /* bad dimension / null pointer */
#define BHI_EBATCH   (-2)   /* batch > BHI_MAX_BATCH (reference: STD_TORCH_CHECK, kernel.cu:472,737) */
#define BHI_ELAYOUT  (-3)   /* table size or chunking does not match the stream format */

#define BHI_MAX_BATCH 8

/* Format and kernel constants, so that host code has one source of truth
 * (the reference duplicates OP_PER_LANE / ANS_PRECISION in functional.py:15-16 and
 * kernel.cu:22-25).  Fills out[0..n) with, in order:
 *   0 format version        1 lanes per wavefront (64)   2 rows per row group (4)
 *   3 columns per step (128)4 Huffman table index bits   5 window words per lane (3)
 *   6 dummy bits per lane   7 max fused batch            8 rANS precision bits
 *   9 stream alignment in 32-bit words                   10 tail padding words
 *  11 task target used by bhi_chunks_per_group           12 max steps per task
 *  13 sizeof(bhi_gemv_member): a binding checks its own struct against it before it
 *     passes arrays of members (the struct has grown once, by its last field)
 * Returns the number of constants available. */
int bhi_constants(int32_t* out, int n);

/* Number of independent streams (chunks) a (split, row group) is cut into; a pure
 * function of the shape shared by encoder, decoder and launch geometry. */
int bhi_chunks_per_group(int M, int Ks, int split_k);

const char* bhi_last_error_string(void);

/* gemv_bf16_huffman(A_rem, A_exp, X, Y!, offsets, LUT1, LUT2, LUT3, LUT4, code_lengths)
 * reference: kernel.cu:445-507 (launcher), :419-442 and :46-219 (kernel).
 *   A_rem   uint8  [split_k, M, Ks]  sign/mantissa plane, lane-ordered
 *   A_exp   int32  [exp_words]       task streams (exp_words includes the tail pad)
 *   X       bf16   [batch, split_k*Ks]
 *   Y       bf16   [batch, M]        written
 *   offsets int32  [split_k, M]
 *   LUT1    uint8  [lut1_bytes]      pair decode table, lut1_bytes = 4 << table bits (8192)
 *   LUT2..4 uint8 [256] (carried for the op signature; not read)
 *   code_lengths uint8 [256]        format header: version, table bits, ESC length, has-escapes */
int bhi_gemv_bf16_huffman(const void* A_rem, const void* A_exp, int64_t exp_words,
                          const void* X, void* Y, const void* offsets,
                          const void* LUT1, int64_t lut1_bytes,
                          const void* LUT2, const void* LUT3, const void* LUT4,
                          const void* code_lengths,
                          int split_k, int M, int Ks, int batch, void* stream);

/* huffman_decode(A_rem, A_exp, Y!, offsets, LUT1, LUT2, LUT3, LUT4, code_lengths)
 * reference: kernel.cu:534-587 (launcher), :510-531 and :222-310 (kernel).
 *   Y bf16 [M, split_k*Ks] row-major original weight, written. */
int bhi_huffman_decode(const void* A_rem, const void* A_exp, int64_t exp_words,
                       void* Y, const void* offsets,
                       const void* LUT1, int64_t lut1_bytes,
                       const void* LUT2, const void* LUT3, const void* LUT4,
                       const void* code_lengths,
                       int split_k, int M, int Ks, void* stream);

/* huffman_encode(data, LUT, output!, output_lengths!)
 * reference: kernel.cu:613-644 (launcher), :590-610 (kernel).
 *   data    uint8  [n_tasks, n_steps, 64, 8]  exponent bytes in lane order
 *   LUT     uint32 [65537]                    encoder table: code | len<<16, ESC last
 *   output  int32  [n_tasks, out_stride]      one finished task stream per row, written
 *   output_lengths int32 [n_tasks]            words used per task (multiple of 4), written
 * out_stride must be >= bhi_encode_capacity(n_steps). */
int bhi_huffman_encode(const void* data, const void* LUT, void* output, void* output_lengths,
                       int n_tasks, int n_steps, int64_t out_stride, void* stream);

/* Worst-case words one task stream of n_steps steps can occupy. */
int64_t bhi_encode_capacity(int n_steps);

/* gemv_bf16_ans(A_rem, A_exp, X, Y!, offsets, LUT)
 * reference: kernel.cu:714-764 (launcher), :686-711 and :46-219 (kernel).
 *   LUT int32 [256]: (sym<<24)|(freq<<12)|rem, rANS precision 8 (functional.py:286-295). */
int bhi_gemv_bf16_ans(const void* A_rem, const void* A_exp, int64_t exp_words,
                      const void* X, void* Y, const void* offsets, const void* LUT,
                      int split_k, int M, int Ks, int batch, void* stream);

/* ans_decode(A_rem, A_exp, Y!, offsets, LUT)
 * reference: kernel.cu:878-919 (launcher), :851-875 and :222-310 (kernel). */
int bhi_ans_decode(const void* A_rem, const void* A_exp, int64_t exp_words,
                   void* Y, const void* offsets, const void* LUT,
                   int split_k, int M, int Ks, void* stream);

/* ans_encode(data, freq, cum, output!, output_lengths!)
 * reference: kernel.cu:814-848 (launcher), :767-811 (kernel).
 *   freq, cum int32 [256] quantised frequencies (sum 256) and their exclusive prefix. */
int bhi_ans_encode(const void* data, const void* freq, const void* cum,
                   void* output, void* output_lengths,
                   int n_tasks, int n_steps, int64_t out_stride, void* stream);

int64_t bhi_ans_encode_capacity(int n_steps);

/* Fixed-width ("nibble") codec -- no counterpart in the reference.  Every exponent inside
 * [base, base+14] is a 4-bit offset in the task block's rows (row t = step t, column j in
 * bits 4j..4j+3 of the lane's word), nibble 15 sends the exponent to the block's escape
 * list.  Same tensors and meanings as the rANS entry points; LUT int32 [256]: [0] base
 * exponent, [1] nonzero when the matrix has escaped exponents, the rest 0. */
int bhi_gemv_bf16_nibble(const void* A_rem, const void* A_exp, int64_t exp_words,
                         const void* X, void* Y, const void* offsets, const void* LUT,
                         int split_k, int M, int Ks, int batch, void* stream);
int bhi_nibble_decode(const void* A_rem, const void* A_exp, int64_t exp_words,
                      void* Y, const void* offsets, const void* LUT,
                      int split_k, int M, int Ks, void* stream);
int bhi_nibble_encode(const void* data, const void* LUT, void* output, void* output_lengths,
                      int n_tasks, int n_steps, int64_t out_stride, void* stream);
int64_t bhi_nibble_encode_capacity(int n_steps);

/* Grouped fused GEMV: up to 4 weights of one codec that multiply the same X (same
 * split_k and Ks, any M) in ONE launch -- the q/k/v or gate/up projections of a decoder
 * layer.  Replaces cudastream_utils.py:8-47 of the reference, which runs q/k/v on parallel
 * streams to the same end (fewer serial launches per token).  Every member is a complete
 * weight as the single entry points take it, with its own output Y bf16 [batch, M]:
 *   table/table_bytes  LUT1 + its size (Huffman) or LUT int32[256] (rANS, nibble; size unchecked)
 *   header             code_lengths (Huffman); ignored for rANS and nibble
 *   bias               bf16 [M] or NULL: added to the BF16-rounded product and rounded again,
 *                      bit for bit the reference's `output += bias` (functional.py:403-404)
 *                      without its extra launch
 * `members` is a host array that is read before the call returns. */
typedef struct bhi_gemv_member {
    const void* A_rem;
    const void* A_exp;
    int64_t exp_words;
    void* Y;
    const void* offsets;
    const void* table;
    int64_t table_bytes;
    const void* header;
    const void* bias;
    int32_t M;
    int32_t reserved;
    const void* residual;          /* bf16 [batch, M] or NULL: added after the bias, as a separate BF16
                                    * `y + residual` (the residual connection around the layer) would */
} bhi_gemv_member;                 /* 88 bytes: nine 8-byte fields, two ints, one 8-byte field */
int bhi_gemv_bf16_huffman_grouped(const bhi_gemv_member* members, int n_members, const void* X,
                                  int split_k, int Ks, int batch, void* stream);
int bhi_gemv_bf16_ans_grouped(const bhi_gemv_member* members, int n_members, const void* X,
                              int split_k, int Ks, int batch, void* stream);
int bhi_gemv_bf16_nibble_grouped(const bhi_gemv_member* members, int n_members, const void* X,
                                 int split_k, int Ks, int batch, void* stream);

/* Grouped GEMV on a FUNCTION of X, so that the layer in front of the linear needs no kernel
 * (and no round trip through memory) of its own -- the reference runs these as separate
 * PyTorch kernels around its op (functional.py:403-404 is the only fusion point it has):
 *   x_mode 1  RMSNorm:  h = x * rsqrt(mean(x^2) + eps) * gamma,  x_aux = gamma bf16 [split_k*Ks]
 *   x_mode 2  SwiGLU:   h = silu(gate) * x,                      x_aux = gate  bf16 [batch, split_k*Ks]
 *   x_mode 0  h = x (the plain grouped entry points)
 * batch <= 4.  The roundings are those of bhi_rms_norm / bhi_silu_mul below followed by the
 * plain GEMV: the fused and the unfused sequence give the same bits. */
int bhi_gemv_bf16_huffman_grouped_x(const bhi_gemv_member* members, int n_members, const void* X,
                                    int split_k, int Ks, int batch, int x_mode, const void* x_aux, float eps,
                                    void* stream);
int bhi_gemv_bf16_ans_grouped_x(const bhi_gemv_member* members, int n_members, const void* X,
                                int split_k, int Ks, int batch, int x_mode, const void* x_aux, float eps,
                                void* stream);
/* The same two pieces as kernels of their own (1..4 rows; out may not alias the inputs of
 * bhi_rms_norm): out = bf16(x * r * gamma) with one rounding; out = bf16(bf16(silu(gate)) * up). */
int bhi_rms_norm(const void* X, const void* gamma, void* out, int rows, int K, float eps, void* stream);
int bhi_silu_mul(const void* gate, const void* up, void* out, int64_t n, void* stream);

/* Fused decode + matrix product for 1..32 rows of X (meant for 9..32; up to 8 the GEMV
 * entry points are faster): Y = X W^T (+ bias) with the weights going from the decoder's
 * registers straight into matrix-core instructions.  Replaces the reference's path above
 * eight rows, huffman_decode / ans_decode to a BF16 matrix followed by a dense GEMM
 * (functional.py:405-407, 460-462; kernel.cu:510-587, 851-919), which writes and re-reads
 * 2*M*K bytes per call.  `weight` is one member as the grouped GEMV takes it (Y bf16
 * [batch, M]; bias and residual as there).  Weights with fewer than 2048 row groups are cut along K
 * over several blocks whose partial sums meet in `workspace`: device memory of at least
 * bhi_gemm_workspace_bytes(...) bytes that was ZERO when first handed to the library and is
 * otherwise only touched by these entry points (every launch leaves its counters at zero);
 * launches that may overlap on the GPU must not share a workspace.  It may be NULL when
 * bhi_gemm_workspace_bytes returns 0. */
int bhi_gemm_bf16_huffman(const bhi_gemv_member* weight, const void* X, int split_k, int Ks, int batch,
                          void* workspace, int64_t workspace_bytes, void* stream);
int bhi_gemm_bf16_ans(const bhi_gemv_member* weight, const void* X, int split_k, int Ks, int batch,
                      void* workspace, int64_t workspace_bytes, void* stream);
/* The same product for up to four weights that multiply one X (members as in the grouped GEMV:
 * same codec, split_k and Ks; bias and residual per member), one grid -- what the reference
 * spreads over parallel streams for the sibling projections of a decoder layer
 * (cudastream_utils.py:8-47).  Takes no workspace: a group whose rows together number fewer
 * than 8192 (bhi_gemm_workspace_bytes of the summed M is not 0) is rejected with BHI_EINVAL and
 * its members go through the calls above one by one. */
int bhi_gemm_bf16_huffman_grouped(const bhi_gemv_member* members, int n_members, const void* X, int split_k,
                                  int Ks, int batch, void* stream);
int bhi_gemm_bf16_ans_grouped(const bhi_gemv_member* members, int n_members, const void* X, int split_k,
                              int Ks, int batch, void* stream);
/* Workspace bytes a call with these dimensions needs (0: none); negative on a rejected shape. */
int64_t bhi_gemm_workspace_bytes(int split_k, int M, int Ks, int batch);

/* bhi_gemm_bf16_huffman without a workspace argument -- no counterpart in the reference.  For
 * callers that cannot allocate device memory at all (code under stream capture that has no
 * workspace yet, serving loops and harnesses that forbid it): the partial sums and counters
 * live in an array inside the library's own device image, bhi_gemm_static_workspace_bytes()
 * bytes (1 KiB of counters + 2 MiB) on every GPU the library is loaded on.  A product that
 * needs more (see bhi_gemm_workspace_bytes) is rejected with BHI_EINVAL.  The call allocates
 * and frees nothing.  All calls on one GPU share the one array: calls that may overlap there
 * (different streams) race. */
int bhi_gemm_bf16_huffman_static(const bhi_gemv_member* weight, const void* X, int split_k, int Ks, int batch,
                                 void* stream);
int64_t bhi_gemm_static_workspace_bytes(void);

/* No counterpart in the reference.  bhi_device_init: looks up, on the current device, what the
 * library otherwise looks up at the first call that needs it (the address of the built-in
 * workspace); call it once per device outside any stream capture if the first use of
 * bhi_gemm_bf16_huffman_static may happen under capture.  bhi_gemm_workspace_reset: enqueues a
 * kernel that zeroes a workspace of the fused matrix product (not a memset node, so it may be
 * captured): for a workspace whose last launch failed or was abandoned, whose counters may be
 * non-zero. */
int bhi_device_init(void);
int bhi_gemm_workspace_reset(void* workspace, int64_t workspace_bytes, void* stream);

/* Readers for weights that were compressed by the reference package itself: same tensors
 * as the reference's huffman_decode / ans_decode ops (kernel.cu:534-587, 878-919) IN THE
 * REFERENCE'S OWN LAYOUT (functional.py:129-242: 64 streams per row, LUT1..4 uint8 [256],
 * code_lengths uint8 [256]; rANS LUT int32 [256]).  Y bf16 [M, split_k*Ks] receives the
 * original weight, which can then be compressed again in this library's layout.  Only
 * M >= 1 and Ks % 128 == 0 are required. */
int bhi_reference_huffman_decode(const void* A_rem, const void* A_exp, int64_t exp_words,
                                 void* Y, const void* offsets,
                                 const void* LUT1, const void* LUT2, const void* LUT3, const void* LUT4,
                                 const void* code_lengths,
                                 int split_k, int M, int Ks, void* stream);
int bhi_reference_ans_decode(const void* A_rem, const void* A_exp, int64_t exp_words,
                             void* Y, const void* offsets, const void* LUT,
                             int split_k, int M, int Ks, void* stream);

/* No counterpart in the reference (which leaves attention to the model code around its linear
 * layers): the attention step of ONE new token of a decoder layer in one launch, so that a
 * recorded decode step is not dominated by small kernels between this library's launches.
 * Per head: RMSNorm of the projected q and k heads (fp32, then times `norm_weight` -- bf16
 * [q_heads + kv_heads, head_dim], or NULL), rotation by the angles of the token's position
 * (`cos`, `sin`: fp32 [max_len, head_dim]; out = x * cos + swap_halves(x) * sin, so `sin` holds
 * -sin in its first half and +sin in its second), k and v written to slot `*pos` of the caches
 * (bf16 [kv_heads, max_len, head_dim]), then softmax(q . k * scale) over slots 0 .. *pos times v
 * for each q head (q heads h * q_heads / kv_heads .. share k/v head h), `out` bf16
 * [q_heads, head_dim].  `qk` is bf16 [q_heads + kv_heads, head_dim] (q heads first), `v` bf16
 * [kv_heads, head_dim]; `pos` points to one int64 in DEVICE memory (a recorded graph follows
 * it); head_dim must be 128, max_len at most 8192.  q, k, the softmax weights and the output
 * are rounded to BF16 where a chain of BF16 torch operations would round them. */
int bhi_decode_attention(const void* qk, const void* v, const void* norm_weight, const void* cos, const void* sin,
                         const void* pos, void* k_cache, void* v_cache, void* out, int q_heads, int kv_heads,
                         int head_dim, int max_len, float eps, float scale, void* stream);

/* No counterpart in the reference: a measurement helper.  Enqueues a kernel in which
 * `wavefronts` wavefronts (a positive multiple of 4) each load a contiguous span of `src`
 * (four 16-byte loads in flight per lane, with or without the non-temporal hint) and keep
 * nothing: the rate at which this GPU feeds a kernel of the fused GEMV's shape when there is
 * nothing to decode.  `src` must be 16-byte aligned; `sink` is 4 bytes of device memory that
 * are not written in practice.  Returns the number of bytes the launch reads (`bytes` rounded
 * down to whole 1 KB loads of every wavefront), or a negative error. */
int64_t bhi_stream_read(const void* src, int64_t bytes, int wavefronts, int nontemporal, void* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* BHI_H */
