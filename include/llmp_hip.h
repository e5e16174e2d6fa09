/*
 * C ABI of the MI355X (gfx950) kernels for llmpalooza's quantized linear-layer
 * path. One enqueue-only launch per operation on a caller-owned hipStream_t
 * (passed as void*): nothing here allocates, synchronizes or frees; every
 * operand and scratch area is the caller's, and stays mapped until a fence
 * after the launch has completed (src/kernels/ggml/launch.h:4-48,
 * src/kernels/decode/products.h:48-51 of the reference).
 *
 * Return values follow src/kernels/ggml/mxfp8_cutlass.h:75-79:
 *    0  queued;
 *   >0  refused before anything was queued (the caller's kRejected);
 *   <0  the runtime reported an error after work may have been queued (the
 *       caller's kUnknown: it faults its launch context).
 * llmp_hip_last_error() names the reason of the calling thread's last
 * non-zero return.
 *
 * Sizes are bytes unless a comment says blocks or elements. "Q8_1 block" is
 * {f16 d; f16 s; i8 qs[32]} = 36 bytes; Q8_0 is {f16 d; i8 qs[32]} = 34 bytes;
 * Q4_K is {f16 d; f16 dmin; u8 scales[12]; u8 qs[128]} = 144 bytes
 * (src/format/encoding.cc:110-116); the legacy blocks are {f16 d; [f16 m;] [u32 high bits;] u8
 * nibbles[16]} = 18 (Q4_0), 20 (Q4_1), 22 (Q5_0), 24 (Q5_1) bytes, code i the low (i < 16) or
 * high nibble of byte i % 16 plus 16 where bit i of the high bits is set
 * (tests/unit/dsv4_fast_test.cc:141-164); MXFP4 is {e8m0 e; u8 nibbles[16]} = 17 bytes, value
 * i the E2M1 value of the low (i < 16) or high nibble of byte i % 16, times 2^(e - 127)
 * (src/format/encoding.cc:130-138, src/kernels/reference/decode.cc:239-248 and 417-428); IQ4_NL is
 * Q4_0's 18 bytes with each nibble an index into ggml's codebook of sixteen int8 values, a value d times the
 * entry (src/format/encoding.cc:126, src/kernels/ggml/vecq.cu:375-396); Q5_K is {f16 d; f16 dmin; u8 scales[12];
 * u8 qh[32]; u8 qs[128]} = 176 bytes, Q4_K with bit g of qh's byte i as the fifth bit of value i of sub-block g
 * (src/format/encoding.cc:116); Q6_K is {u8 ql[128]; u8 qh[64]; i8 scales[16]; f16 d} = 210 bytes, value
 * 128 h + 32 t + l the nibble t / 2 of ql[64 h + 32 (t % 2) + l] plus 16 times bits 2t, 2t + 1 of qh[32 h + l], minus 32,
 * times scales[value / 16] times d (src/format/encoding.cc:117).
 */
#ifndef LLMP_HIP_H_
#define LLMP_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml_type values of the weight encodings the kernels read. */
enum { LLMP_TYPE_Q4_0 = 2, LLMP_TYPE_Q4_1 = 3, LLMP_TYPE_Q5_0 = 6, LLMP_TYPE_Q5_1 = 7, LLMP_TYPE_Q8_0 = 8, LLMP_TYPE_Q4_K = 12, LLMP_TYPE_MXFP4 = 39, LLMP_TYPE_IQ4_NL = 20, LLMP_TYPE_Q5_K = 13, LLMP_TYPE_Q6_K = 14 };
/* VecQGlu, src/kernels/ggml/llmp_ops.h:1072. */
enum { LLMP_GLU_NONE = 0, LLMP_GLU_SWIGLU = 1, LLMP_GLU_SWIGLU_CLAMP = 2, LLMP_GLU_GEGLU = 3 };
/* Element types of unquantized activations. */
enum { LLMP_X_F32 = 0, LLMP_X_BF16 = 1, LLMP_X_F16 = 2 };

const char* llmp_hip_last_error(void);
/* Compute units of the current device (the `sms` argument of the reference's
 * Scratch/Run pairs). Negative on a runtime error. */
int llmp_hip_compute_units(void);

/* ------------------------------------------------------------------ llmp.q8_1
 * Replaces quantize_row_q8_1_cuda as RunQuantizeQ8 calls it
 * (src/kernels/ggml/vecq.cu:1095-1111; dispatch shape in
 * third_party/patches/ggml/0010-llmp-q8-dispatch-descriptors.patch:604-611).
 * x: rows x planes rows of k floats, row_stride / plane_stride floats apart.
 * out: for each plane then row, padded_k / 32 Q8_1 blocks; blocks past k are zero.
 * padded_k is k rounded up to 512 (src/kernels/ggml/llmp_ops.cc:2574-2576). */
int llmp_hip_q8_1_quantize(const float* x, void* out, int64_t k, int64_t padded_k,
                           int64_t row_stride, int64_t rows, int64_t planes, int64_t plane_stride,
                           void* stream);

/* ------------------------------------------------------------------ llmp.vecq
 * The POD of src/kernels/ggml/vecq.h:22-41, field for field. Weight offsets
 * count the weight type's blocks; activation offsets count Q8_1 blocks. */
typedef struct llmp_vecq_desc {
  const void* w;      /* weights (the up projection with a GLU) */
  const void* g;      /* gate weights, or null */
  const void* y;      /* Q8_1 activations */
  const int32_t* ids; /* null: dense or grouped */
  float* dst;
  int ncols_x;       /* k */
  int nrows;         /* n */
  int stride_row;    /* weight blocks between rows */
  int stride_expert; /* weight blocks between experts */
  int y_token;       /* Q8_1 blocks between tokens' rows */
  int y_slot;        /* between slots' rows (per-slot activations), else 0 */
  int ids_stride;    /* ids between tokens */
  int used;
  int tokens;
  int dst_token; /* floats */
  int dst_slot;
  int glu; /* LLMP_GLU_* */
  float limit;
} llmp_vecq_desc;

/* Replaces LaunchVecQ (src/kernels/ggml/vecq.h:43-47, vecq.cu:1023-1094):
 * variant -1 is the default for the shape; returns 1 for a variant the shape
 * cannot take, as the reference returns false. tokens 1..16, used * tokens
 * <= 128 when routed (src/kernels/ggml/llmp_ops.cc:2931-2948). */
int llmp_hip_vecq(int type, const llmp_vecq_desc* d, int variant, void* stream);
int llmp_hip_vecq_variants(void);
const char* llmp_hip_vecq_variant_name(int variant);

/* An import-time relayout for this device, lossless and undone by inverse != 0 (the reference does its
 * platform-specific relayouts at import, src/import/expert_relayout.h:4-17: a table rewritten into the tile order
 * its products read). Q4_K rows (nrows x blocks_per_row super-blocks, packed) in tiles of 64 rows: within a tile
 * the blocks lie super-block after super-block, a super-block's 64 rows together, so that the 9216 bytes a wave of
 * the row-a-lane product reads at a time are consecutive (over the reference's row-major blocks that read fetches
 * 1.3 to 1.4 times its bytes: 144-byte pieces are ragged against HBM's 64-byte units). A 64-row tile covers the same
 * bytes in both layouts, so a table of experts or matrices is relaid out in one call (nrows = all its rows) as long
 * as every matrix is whole tiles. llmp_hip_vecq's variant "rows pass8 tiles64" reads the result; every other variant
 * reads the reference's layout. src and dst at 16-byte boundaries, not overlapping. */
int llmp_hip_relayout_q4_k_tiles64(const void* src, void* dst, int64_t nrows, int64_t blocks_per_row, int inverse, void* stream);
/* The same for Q8_0 rows (nrows x blocks_per_row blocks of 34 bytes, packed; blocks_per_row a multiple of four), the
 * split the reference's importer notes call for (codes and scales apart, the codes at 16-byte boundaries): a tile's
 * piece is four blocks of each of its 64 rows, 8704 bytes: the rows' codes (row r's 128 at 128 r, its 16-byte chunk c
 * at place c ^ (r % 8), so that lanes reading one chunk of eight rows use every bank of LDS once), then the rows' four
 * F16 scales, 8 bytes a row. The same bytes in all, lossless, undone by inverse != 0. llmp_hip_vecq's variant
 * "rows pass8 tiles64" reads it for Q8_0 products of 2 to 8 tokens (a weight row a lane on the 4 x 4 x 4 int8 matrix
 * instruction, the weights read once: where the reference's layout goes through the four-token passes or the
 * 16-token matrix form, 1.3 to 1.7 times slower at 4 to 8 tokens). The rows at 2-byte, the tiles at 16-byte
 * boundaries (inverse: the other way round), not overlapping. */
int llmp_hip_relayout_q8_0_tiles64(const void* src, void* dst, int64_t nrows, int64_t blocks_per_row, int inverse, void* stream);

/* The same product over unquantized activations: each workgroup quantizes the
 * tokens' rows to Q8_1 in LDS (the arithmetic of llmp_hip_q8_1_quantize, bit
 * for bit) instead of reading d->y, which is ignored. x_token / x_slot are
 * elements between tokens' and slots' rows (x_slot 0: every slot reads the
 * token's row). This is the reference's in-kernel activation quantization
 * (src/kernels/ggml/llmp_moe.cu:469-571) for the GGML block types. */
typedef struct llmp_vecq_source {
  const void* x;
  int x_type; /* LLMP_X_* */
  int64_t x_token;
  int64_t x_slot;
} llmp_vecq_source;
int llmp_hip_vecq_fused(int type, const llmp_vecq_desc* d, const llmp_vecq_source* x, int variant,
                        void* stream);

/* Test aid: the int32 sums of every (row, block) of a dense one-token product
 * as the kernel's integer path computes them, added into `sums` (which the
 * caller zeroes first): sums[(row * blocks + b) * per + i] with per = 1 for
 * Q8_0 (sum of w * q) and 16 for Q4_K (eight sub-block sums of code * q, then
 * eight of q; tests/unit/dsv4_fast_test.cc:185-191). */
int llmp_hip_vecq_block_sums(int type, const llmp_vecq_desc* d, int variant, int32_t* sums,
                             void* stream);

/* llmp.vecq over rows sorted by expert (the grouped form of a routed product with more
 * than 128 (token, slot) pairs; src/kernels/decode/products.h:151-169 and
 * src/kernels/ggml/moe_cutlass.h:12-27 describe the reference's operand layout): expert e
 * computes rows offsets[e] .. offsets[e + 1] of the Q8_1 activations d->y (y_token blocks a
 * row) into the same rows of d->dst (dst_token floats a row) with matrix e of d->w / d->g.
 * d->ids, used, tokens and the slot strides are ignored. Weights the flat or the matrix-core
 * form takes (the rows form has no sorted variant). */
int llmp_hip_vecq_sorted(int type, const llmp_vecq_desc* d, const int32_t* offsets, int experts,
                         int variant, void* stream);

/* ------------------------------------------------------------------ routed experts
 * llmp.moe.router (src/kernels/ggml/llmp_fused.cu:1307-1407; the definition is kRoute with
 * kSoftmaxTopK, src/kernels/reference/exec.cc:1728-1818): per token the softmax of its
 * `experts` logits, the `used` most probable experts (the lower index first among equals; a
 * row holding a NaN or no finite value picks experts 0 .. used - 1 with zero weights), and
 * their probabilities, over max(their sum, 2^-14) when `normalize`, times `scale`.
 * logits [tokens][experts] -> ids, weights [tokens][used]. used <= 64, experts <= 1024. */
int llmp_hip_moe_router(const float* logits, int experts, int used, int tokens, int normalize,
                        float scale, int32_t* ids, float* weights, void* stream);

/* llmp.moe.route (src/kernels/ggml/llmp_moe.cu:81-163): ids [tokens][used] (ids_stride
 * apart) into the route buffer of src/kernels/ggml/moe_layout.h:46-70, int32, in this order:
 * offsets[experts + 1], scale_rows[experts + 1], position[slots], token[slots],
 * expert[slots], counts[chunks * experts] (work space; chunks = ceil(tokens / 64)). Rows are
 * sorted by expert, token order within an expert; an id outside the experts has position -1. */
int64_t llmp_hip_moe_route_ints(int experts, int used, int tokens);
int llmp_hip_moe_route(const int32_t* ids, int ids_stride, int experts, int used, int tokens,
                       int32_t* route, void* stream);

/* One token through a routed-expert FFN layer (Q4_K experts) in one or two launches: llmp.moe.router, the picked experts'
 * gate/up products with their GLU, their down products and the ordered weighted sum, which the reference's graph holds
 * as kRoute, kMatMulId, kGlu, kMatMulId and kExpertReduce (src/ir/decompose.cc:1080-1109) and the entry points above
 * run as four launches. It has no single counterpart in the reference: it is those operations fused for the decode
 * step, where each launch costs more than its bytes. Results are bit for bit llmp_hip_moe_router's ids and weights
 * and llmp_hip_vecq_fused (gate/up with the GLU; down) followed by llmp_hip_moe_combine.
 * logits F32 [experts]; x the token's `hidden` activations (x_type LLMP_X_F32 or LLMP_X_BF16); gate_up: an expert's
 * 2 * ffn rows of `hidden` values, the gate's rows first, gate_up_stride blocks an expert; down: hidden rows of ffn
 * values, down_stride blocks an expert; out F32 [hidden]; ids, weights [used]: the router's result, written; h F32
 * [used][ffn]: scratch for the activated values (llmp_hip_moe_token_scratch bytes). used <= 8, hidden and ffn whole
 * super-blocks (hidden <= 8192).
 * launches 1: the two halves meet inside the launch at `sync`, 16 + 4 * cus bytes of device memory that are zero
 * before their first use and need no reset between calls or graph replays with the same `cus` (each workgroup keeps
 * the number of meetings it has come to in a word of its own from byte 16 on); word 2 of it is set to 1 if
 * a workgroup ever gave up waiting (the results of that call are then wrong; it never happens while the whole grid,
 * `cus` workgroups, is resident, which takes a device this call has to itself: no other kernel of another stream
 * holding compute units for long). launches 2: the same two halves as two launches, `sync` unused: the faster of the
 * two on an MI355X (16.7 us against 19.3 at 128 experts, top 8, hidden 2048, ffn 768; the four operations 20 us):
 * agent-scope stores and loads take longer to cross the device than a launch boundary does. Calls that share h, ids,
 * weights or sync must not overlap. */
typedef struct llmp_moe_token {
  const float* logits;
  const void* x;
  const void* gate_up;
  const void* down;
  float* out;
  int32_t* ids;
  float* weights;
  float* h;
  void* sync;
  int64_t gate_up_stride, down_stride; /* blocks an expert */
  int32_t type;                        /* LLMP_TYPE_Q4_K */
  int32_t x_type;
  int32_t experts, used, hidden, ffn;
  int32_t glu;       /* LLMP_GLU_* */
  int32_t normalize; /* the router's: weights over their sum */
  float limit, route_scale;
} llmp_moe_token;
size_t llmp_hip_moe_token_scratch(const llmp_moe_token* op);
int llmp_hip_moe_token(const llmp_moe_token* op, int launches, int cus, void* stream);

/* llmp.q8_1 with a gather, quantize_row_q8_1_cuda's `ids` argument
 * (third_party/patches/ggml/0010-llmp-q8-dispatch-descriptors.patch:604-611): output row r
 * is the Q8_1 of input row rows[r] (row r when rows is null), row_stride floats apart. */
int llmp_hip_q8_1_quantize_rows(const float* x, const int32_t* rows, void* out, int64_t k,
                                int64_t padded_k, int64_t row_stride, int64_t count, void* stream);

/* The routed rows' weighted sum (kExpertReduce, src/kernels/reference/exec.cc:1819-1856;
 * src/kernels/ggml/llmp_fused.cu:200-240 and llmp_moe.cu:390-427 for sorted rows):
 * out[t][:] = sum_j x[row(t, j)][:] * weights[t][j] in slot order, the first term assigned,
 * where row(t, j) is t * used + j, or position[t * used + j] when position is given (a
 * negative position adds nothing). width a multiple of 4. */
int llmp_hip_moe_combine(const float* x, const float* weights, const int32_t* position, int width,
                         int used, int tokens, float* out, void* stream);

/* ------------------------------------------------------------------ MXFP8
 * E4M3 codes with one E8M0 scale per 32 values along K. "Atoms" is the scale layout of
 * src/format/layout.h:108-113 (ScaleAtomOffset; the same as moe_cutlass.h:42-46 SfOffset):
 * 128-row by 4-scale atoms of 512 bytes, along K first, rows padded to 128, k a multiple of 128.
 *
 * llmp.mxfp8.quantize (src/kernels/ggml/llmp_ops.cu:610-648, mxfp8_quant.cuh:19-46): rows of
 * k F32 or BF16 values, x_stride elements apart, to codes [rows][k] and scales in atoms for
 * the rows rounded up to 128 (the padding rows' scales zero): RowsLayout of
 * mxfp8_cutlass.h:42-57 with the two parts passed separately. */
int llmp_hip_mxfp8_quantize(const void* x, int x_type, int64_t x_stride, int64_t k, int64_t rows,
                            void* codes, void* scales, void* stream);
/* llmp.mxfp8.swizzle (llmp_ops.cu:652-663): a weight's scales [n][k / 32] into atoms. */
int llmp_hip_mxfp8_swizzle(const void* scales, int64_t n, int64_t k, void* out, void* stream);
/* llmp.mxfp8.mul_mat_vec (llmp_ops.cu:145-224): y[t][r] = sum over blocks of (sum of 32
 * E4M3(code) * x) * 2^(scale - 127), scales plain [n][k / 32], x F32 [tokens][k], 1..16
 * tokens, y F32 [tokens][n]. */
int llmp_hip_mxfp8_gemv(const void* codes, const void* scales, int64_t n, int64_t k, const float* x,
                        int tokens, float* y, void* stream);

/* llmp.mxfp8.gemm: mxfp8::Gemm / Available / Scratch / Run of
 * src/kernels/ggml/mxfp8_cutlass.h:56-79, field for field. D[m, n] = A[m, k] * B[n, k]^T,
 * both operands codes with scales in atoms, F32 accumulation, D F32 or BF16 (rounded once). */
typedef struct llmp_mxfp8_gemm {
  int m;
  int n;
  int k;
  const void* a;        /* codes, m rows of k */
  const void* a_scales; /* atoms */
  const void* b;        /* codes, n rows of k */
  const void* b_scales; /* atoms */
  void* d;              /* m rows of n */
  unsigned char bf16;   /* one byte, as the reference's `bool bf16` (mxfp8_cutlass.h:67): non-zero is D in
                           BF16, else F32; the seven bytes of padding after it are never read */
  void* scratch;        /* llmp_hip_mxfp8_gemm_scratch bytes, 256-byte aligned (none needed: may be null) */
} llmp_mxfp8_gemm;
int llmp_hip_mxfp8_gemm_available(void);
size_t llmp_hip_mxfp8_gemm_scratch(const llmp_mxfp8_gemm* gemm, int compute_units);
/* `compute_units` (the reference's `sms`; 0 or less: 256): the launch has at most that many workgroups, each going
 * through its share of the tiles one after the other. The sums do not depend on it. */
int llmp_hip_mxfp8_gemm_run(const llmp_mxfp8_gemm* gemm, int compute_units, void* stream);

/* ------------------------------------------------------------------ llmp.moe.gemm
 * moe::GroupedGemm / GroupedGemmAvailable / GroupedGemmScratch / RunGroupedGemm of
 * src/kernels/ggml/moe_cutlass.h:48-76, field for field: the block-scaled NVFP4 grouped GEMM over routed rows
 * sorted by expert. One group an expert e: D_e[M_e, n] = A_e[M_e, k] B_e[n, k]^T, F32 accumulation, D BF16.
 * A holds every routed row: expert e's rows are rows offsets[e] .. offsets[e + 1] of the codes (E2M1, k / 2 bytes
 * a row, element 2i in the low nibble); its UE4M3 scales (one per 16 elements) lie in the atoms of
 * moe_cutlass.h:42-46 (SfOffset, k / 16 scales a row) in a block of rows starting at sf_rows[e] (a multiple of
 * 128, as llmp_hip_moe_route's scale_rows). B_e is at weights + e * expert_stride: n rows of codes at
 * codes_offset, their scales at scales_offset in the atoms of n rows. offsets and sf_rows are device arrays of
 * groups + 1 entries. k a multiple of 64; the codes (a, weights, expert_stride, codes_offset) at 16-byte and the
 * scales (a_scales, scales_offset) at 4-byte boundaries. The scratch is not used (llmp_hip_grouped_gemm_scratch is 0: may be
 * null). Values are the format's own: E2M1 times UE4M3 is exact in F16, the products run on the F16 matrix
 * instructions (this device's scaled instructions take E8M0 scales per 32, not UE4M3 per 16). */
typedef struct llmp_grouped_gemm {
  int groups;
  int n;
  int k;
  const int32_t* offsets;
  const int32_t* sf_rows;
  const void* a;
  const void* a_scales;
  const void* weights;
  uint64_t expert_stride;
  uint64_t codes_offset;
  uint64_t scales_offset;
  void* d;
  void* scratch;
} llmp_grouped_gemm;
int llmp_hip_grouped_gemm_available(void);
size_t llmp_hip_grouped_gemm_scratch(int groups, int compute_units);
int llmp_hip_grouped_gemm_run(const llmp_grouped_gemm* gemm, int compute_units, void* stream);

/* ------------------------------------------------------------------ KV cache store
 * llmp.set_rows.quant (SetRowsQuant, src/kernels/ggml/kv_quant.h:28-60,150-158): `rows` rows of k
 * F32 values (k a multiple of 32, x_stride floats apart, 16-byte aligned) stored as rows
 * ids[r] (I32 or I64 by index_bytes) of a Q8_0 or Q4_0 destination whose rows are row_bytes
 * apart. Each block of 32 is quantized with the arithmetic of src/kernels/ggml/kv_quant.cuh:27-69
 * (GGML's reference quantizers, every step an IEEE operation). The two-dimensional case of
 * ggml_set_rows's shapes only: one plane, one batch, no broadcast of the indices (the reference's
 * kv_quant_store.cu:27-58 also takes planes and batches; a caller with per-head planes makes one call a
 * plane, or one grouped call of up to sixteen). `cells` is the destination's number of rows, by which the
 * call refuses a destination that overlaps the values or the indices. Indices are the caller's to bound
 * (kv_quant.h:62-63). */
int llmp_hip_set_rows_quant(int type, const float* x, int64_t x_stride, const void* ids, int index_bytes,
                            void* destination, int64_t row_bytes, int64_t k, int64_t rows, int64_t cells,
                            void* stream);

/* llmp.set_rows.grouped_quant (SetRowsQuantGroup, src/kernels/ggml/kv_quant.h:82-84, 172-178;
 * src/kernels/ggml/kv_quant.cc:214-236): two to sixteen such stores in one launch (a layer's K and V rows, or
 * several layers'), each as llmp_hip_set_rows_quant takes it; `cells` is the destination's number of rows, by
 * which the call refuses a destination that overlaps another store's destination, values or indices. */
typedef struct llmp_set_rows_store {
  int type;        /* LLMP_TYPE_Q8_0 or LLMP_TYPE_Q4_0 */
  int index_bytes; /* 4 or 8 */
  const float* x;
  int64_t x_stride;
  const void* ids;
  void* destination;
  int64_t row_bytes;
  int64_t k;
  int64_t rows;
  int64_t cells;
} llmp_set_rows_store;
int llmp_hip_set_rows_quant_group(int count, const llmp_set_rows_store* stores, void* stream);

/* llmp.rope.set_rows_quant (RopeSetRowsQuant, src/kernels/ggml/kv_quant.h:180-192; the kernel's arithmetic
 * src/kernels/ggml/kv_quant_rope.cu:29-120): a forward NEOX RoPE of `tokens` rows of `heads` heads of head_dim F32
 * values (the first n_dims channels of a head rotate, channel c with c + n_dims / 2; the rest pass through), each
 * token's rotated row quantized into row ids[token] of a Q8_0 or Q4_0 destination [cells][heads * head_dim]. The
 * angle of pair p at position pos[token] is pos * theta_scale^p / freq_factors[p] (theta_scale = freq_base^(-2 /
 * n_dims), kv_quant.cc:383), scaled by freq_scale, or YaRN's mix of both between corr_dims where ext_factor is not
 * zero; cosine and sine are scaled by attn_factor (times 1 + 0.1 ln(1 / freq_scale) under YaRN). The rotated
 * values are F32 results of this device's cosf, sinf and powf: stored codes equal those of a rotation computed in
 * FP64 except where a value lies within that error of a rounding boundary. */
typedef struct llmp_rope_store {
  int type;                  /* LLMP_TYPE_Q8_0 or LLMP_TYPE_Q4_0 */
  int heads, head_dim, n_dims;
  const float* x;
  int64_t x_head_stride;     /* floats */
  int64_t x_token_stride;    /* floats */
  const int32_t* pos;        /* a position a token */
  const float* freq_factors; /* n_dims / 2 of them, or null */
  const int64_t* ids;        /* a destination row a token */
  void* destination;
  int64_t row_bytes;
  int64_t tokens;
  float freq_scale, ext_factor, attn_factor, theta_scale;
  float corr_dims[2];
} llmp_rope_store;
int llmp_hip_rope_set_rows_quant(const llmp_rope_store* store, void* stream);

/* ggml.flash_attn_ext.vec_q8_0 / vec_q4_0 (FlashAttnVecQuant over a checked ggml_flash_attn_ext node,
 * src/kernels/ggml/kv_quant.h:9-26, 146-160; the checks of src/kernels/ggml/kv_quant.cc:81-170): attention that
 * reads K and V as the Q8_0 or Q4_0 blocks the stores above wrote, nothing expanded into device memory.
 * Q F32, value (d, row, head) at q[d + row * q_row_stride + head * q_head_stride] (ggml's [D, rows, heads]); K
 * and V of one block type, the row of (cell, KV head) at cell * cell_stride + head * head_stride bytes (whole
 * blocks; the reference's view [D, cells, KV heads] of a cache that holds a cell's heads together); an F16 mask
 * row of `cells` values a query row, added to the scaled scores (-inf hides a cell); optional F32 sinks, one a
 * head, in the softmax's denominator; output F32 [rows][heads][D] (ggml's [D, heads, rows]). head_dim 64 or 256
 * (512 for Q8_0), cells a multiple of 256, heads a multiple of kv_heads by at most 8, a positive finite scale,
 * softcap 0 or a positive one at head_dim 256 (score = softcap * tanh(score / softcap) before the mask), no
 * ALiBi. The queries pass through Q8_1 for the K product, as in the reference's kernel; sums are F32. A query
 * row that sees no cell (and has no sink) is zeros. The cells are split over workgroups whose partial results go
 * through `scratch` (llmp_hip_attn_vec_quant_scratch bytes for the same `cus`, the device's compute units; 0
 * where the operands would be refused) and are combined by a second launch. Returns as the launchers above. */
typedef struct llmp_attn_vec_quant {
  const void* q;
  const void* k;
  const void* v;
  const void* mask;
  const void* sinks; /* or NULL */
  void* out;
  int64_t q_row_stride, q_head_stride; /* floats */
  int64_t k_cell_stride, k_head_stride, v_cell_stride, v_head_stride; /* bytes */
  int64_t mask_row_stride; /* halves */
  int32_t type; /* LLMP_TYPE_Q8_0 or LLMP_TYPE_Q4_0 */
  int32_t head_dim, heads, kv_heads, rows, cells;
  float scale, softcap;
} llmp_attn_vec_quant;
size_t llmp_hip_attn_vec_quant_scratch(const llmp_attn_vec_quant* op, int cus);
int llmp_hip_attn_vec_quant(const llmp_attn_vec_quant* op, void* scratch, size_t scratch_bytes, int cus, void* stream);

/* ------------------------------------------------------------------ EXL3
 * The trellis-coded linear. Weights as src/kernels/exl3/validate.h:84-96 holds them: the
 * trellis [k / 16][n / 16][16 * bits] uint16, suh (k F16) and svh (n F16); every dimension a
 * multiple of 128. The codebook is a parameter (src/format/encoding.h:121 of the reference):
 * the reference's device kernels build MCG only, its CPU definition all three
 * (src/kernels/reference/decode_exl3.cc:41-66). */
enum { LLMP_EXL3_3INST = 0, LLMP_EXL3_MCG = 1, LLMP_EXL3_MUL1 = 2 };
typedef struct llmp_exl3_weights {
  const void* trellis;
  const void* suh;
  const void* svh;
  int k;
  int n;
  int bits;
  int codebook; /* LLMP_EXL3_* */
} llmp_exl3_weights;

/* LaunchContext::Reconstruct, unfused (src/kernels/exl3/launch.h:100-103, validate.h:186-197):
 * columns [column, column + columns) of the weights in the rotated basis into w
 * (k x columns F16, row-major); whole 16-column tiles. */
int llmp_hip_exl3_reconstruct(const llmp_exl3_weights* weights, void* w, int column, int columns,
                              void* stream);

/* LaunchContext::Reconstruct with ReconstructOperands::fused (src/kernels/exl3/launch.cc:425-448, validate.h:183-193;
 * the definition src/kernels/reference/decode.h:37-43): the same columns of the weights themselves,
 * W = diag(suh) H What H diag(svh) / 128 with H the 128-point transform over each block of 128 inputs and of 128
 * outputs, into w (k x columns F16, row-major, at a 16-byte boundary), for the reconstruction path's plain GEMM from
 * 1,024 rows. Whole 128-column blocks. The transforms run in F32 and a value is rounded to F16 once (the
 * reference's kernel rounds every butterfly to F16). */
int llmp_hip_exl3_reconstruct_fused(const llmp_exl3_weights* weights, void* w, int column, int columns,
                                    void* stream);

/* LaunchContext::Hadamard (launch.h:104-106, validate.h:199-212): 128-point Hadamard
 * transforms of the rows of x (rows x columns) into y (x itself or disjoint), times
 * 1 / sqrt(128): F16 with the input scale (y = H(x * scale)), or F16 / F32 with the output
 * scale (y = H(x) * scale). scale: columns F16. */
int llmp_hip_exl3_hadamard(const void* x, void* y, const void* scale, int rows, int columns, int f32,
                           int input_scale, void* stream);

/* The packed linear: LinearOperands of validate.h:118-131 and PackedGemvLinear / PackedGemmLinear of
 * src/kernels/exl3/linear.h:47-54, 1 to 65536 rows (validate.h:76) in passes of sixteen, each pass streaming
 * the weights once (upstream's choice, validate.h:254-256, is this path through 144 rows and the
 * reconstruction above, which is not built: a caller with more rows pays a pass every sixteen). x (m x k F16)
 * into y (m x n, F16 or F32); a_had is the caller's m x k F16 scratch for the transformed input, which the
 * launches write as they compute it. `scratch` (llmp_hip_exl3_linear_scratch bytes, 8-byte aligned: one pass's,
 * shared by the passes in stream order) takes the place of the reference's lock area: the K slices' partial
 * sums, added in slice order. Two launches a pass are queued (three above four rows: the input transform is
 * then a launch of its own); a failure after the first is reported as a fault (negative). */
typedef struct llmp_exl3_linear {
  llmp_exl3_weights weights;
  const void* x;
  void* a_had;
  void* y;
  int f32; /* y in F32, else F16 */
  int m;
} llmp_exl3_linear;
size_t llmp_hip_exl3_linear_scratch(const llmp_exl3_linear* op);
int llmp_hip_exl3_linear(const llmp_exl3_linear* op, void* scratch, size_t scratch_bytes, void* stream);

/* The same linear for callers that cannot allocate or bring a workspace (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc). It has no counterpart in the reference, whose callers always
 * declare and charge their workspace (src/kernels/ggml/launch.h:4-8). The partial sums go to an array of
 * LLMP_EXL3_STATIC_SCRATCH_BYTES that the library holds on every device it runs on until the process ends; the
 * call allocates and frees nothing. A linear whose llmp_hip_exl3_linear_scratch exceeds that is refused (status
 * 1): pass scratch of your own to llmp_hip_exl3_linear. x, a_had and y are the caller's as before. Every call on
 * a device shares that device's array: calls that overlap in time on one device (two streams) race; calls on one
 * stream, or ordered by events, are safe. Nothing in the array needs clearing: every launch overwrites the part
 * it later reads. Output bits are those of llmp_hip_exl3_linear. */
#define LLMP_EXL3_STATIC_SCRATCH_BYTES ((size_t)4 << 20) /* config 5 at 16 rows needs 3,670,016 */
int llmp_hip_exl3_linear_static(const llmp_exl3_linear* op, void* stream);
/* What the first llmp_hip_exl3_linear_static call on a device and for a (codebook, bits) does besides launching:
 * taking the static array's address and asking the runtime once for the product kernels' dynamic LDS. Neither is
 * a launch, so a stream capture may refuse or be invalidated by them: a caller that captures calls this first,
 * outside any capture, with the device current (only op->weights is read; no stream, nothing is queued), or makes
 * its first call of each such linear eagerly. Like its sibling it has no counterpart in the reference. Returns
 * as the launchers do. */
int llmp_hip_exl3_linear_static_prepare(const llmp_exl3_linear* op);

/* The reconstruction paths of one linear (ReconstructedLinear, src/kernels/exl3/linear.h:57-60 and linear.cc:87-190,
 * over ReconstructedOperands, validate.h:263-277; upstream's choice from 145 rows, fused from 1,024): the weights
 * are reconstructed to F16 a slice of up to 32,768 columns at a time into `w` (llmp_hip_exl3_reconstructed_scratch
 * bytes: k x min(n, 32,768) halves, ReconstructScratchBytes) and each slice is multiplied by a plain F16 product with
 * F32 sums into its columns of y. fused: the weights themselves (llmp_hip_exl3_reconstruct_fused's values) times x.
 * Not fused: the rotated weights times the transformed input (written to op->a_had, m x k halves), then the output's
 * transform over y in place. The reference's product is cuBLASLt's (recon_gemm.h); this one is the library's own
 * (the MXFP8 product's loop over F16 operands), which reads both operands along K, so `w` holds a slice column by
 * column (columns x k), not k x columns: it is scratch of this call, not an interface. x, y, w (and a_had) at
 * 16-byte boundaries, apart from each other and from the weights. No bias (the reference's add_kernel_hhh is not
 * built). Results are the linear's definition within F16 rounding of the reconstructed weights (the reference's
 * bound: 2^-8 of a row's RMS), not bit for bit the packed path's. */
size_t llmp_hip_exl3_reconstructed_scratch(const llmp_exl3_weights* weights);
int llmp_hip_exl3_linear_reconstructed(const llmp_exl3_linear* op, void* w, size_t w_bytes, int fused, int compute_units,
                                       void* stream);

/* exl3.multi_linear.mgemm: MultiLinear of src/kernels/exl3/linear.h:51-53 over the operands of
 * src/kernels/exl3/validate.h:160-172, a gate and an up linear of the same k, n and rate over
 * one input (tests/unit/exl3_trellis_test.cc:664-716). x (m x k F16) into y (2 x m x n: the
 * first linear's rows, then the second's); a_had is 2 x m x k F16 (validate.cc:257-260), each
 * linear's own transformed input. The reference's three pointer tables have no counterpart:
 * the launches carry the six addresses. Same launches as llmp_hip_exl3_linear, both linears in
 * each (one linear after the other where their codebooks differ), in the same passes of sixteen rows;
 * `scratch` is llmp_hip_exl3_multi_linear_scratch bytes. */
typedef struct llmp_exl3_multi_linear {
  llmp_exl3_weights first;
  llmp_exl3_weights second;
  const void* x;
  void* a_had;
  void* y;
  int f32; /* y in F32, else F16 */
  int m;
} llmp_exl3_multi_linear;
size_t llmp_hip_exl3_multi_linear_scratch(const llmp_exl3_multi_linear* op);
int llmp_hip_exl3_multi_linear(const llmp_exl3_multi_linear* op, void* scratch, size_t scratch_bytes, void* stream);

/* ---------------------------------------------------------------- llmp.decode.vector
 * RunVector of src/kernels/decode/products.h:96-109: y[t][j] = sum_k W[first + j][k] x[t][k]
 * (times the weight's tensor scale of row first + j) for t < rows (1 to 16) and j < outputs,
 * over a weight in its stored encoding; row t of x (F32, 16-byte aligned, x_stride a multiple
 * of 4 floats) at x + t * x_stride, of y at y + t * y_stride. The decoders are the reference's
 * (src/kernels/decode/operand.h:26-41, decoders.cuh), the operand its Operand
 * (operand.h:74-97) field for field; values decode as src/kernels/reference/decode.cc has
 * them (an undefined block scale, UE4M3 from 0x7F or E8M0 0xFF, is NaN; the affine encoding is
 * s * q + b rounded once, or s * (q - z)). Rows up to 16384 values; four input rows a launch (fewer of long rows),
 * so 1 to 16 launches are queued and a failure after the first is a fault (negative). */
enum {
  LLMP_DECODER_BF16_DENSE = 0,
  LLMP_DECODER_F16_DENSE = 1,
  LLMP_DECODER_Q8_0_BLOCKS = 2,       /* GGML's block_q8_0 */
  LLMP_DECODER_NVFP4_SPLIT = 3,       /* codes k / 2 bytes a row, UE4M3 scales k / 16 a row */
  LLMP_DECODER_NVFP4_ATOMS = 4,       /* codes as split, scales in CUTLASS's SM1xx atoms */
  LLMP_DECODER_NVFP4_INTERLEAVED = 5, /* each row's codes, then its scales */
  LLMP_DECODER_NVFP4_GGML_BLOCKS = 6, /* GGML's block_nvfp4: four scales, then 32 bytes */
  LLMP_DECODER_MXFP8_SPLIT = 7,       /* E4M3 codes k bytes a row, E8M0 scales k / 32 a row */
  LLMP_DECODER_MXFP8_ATOMS = 8,
  LLMP_DECODER_MXFP4_SPLIT = 9,       /* E2M1 codes k / 2 bytes, E8M0 scales k / 32 */
  LLMP_DECODER_MXFP4_ATOMS = 10,
  LLMP_DECODER_AFFINE_SPLIT = 11
};
typedef struct llmp_decode_operand {
  const uint8_t* data;       /* kData, or kCodes for the split arrangements */
  const uint8_t* scales;     /* kBlockScales for the split arrangements */
  const float* tensor_scale; /* or null: row r takes tensor_scale[r / rows_per_scale] */
  const uint8_t* biases;     /* affine only: biases as the scales, or packed zero points */
  uint32_t k;                /* values a row */
  uint32_t rows;             /* rows of the matrix */
  uint32_t rows_per_scale;
  uint32_t pad;
  uint64_t row_bytes;        /* bytes of a row of `data` */
  uint32_t scale_row_bytes;  /* affine only: bytes of a row of `scales` (and of the biases) */
  uint16_t group;            /* affine only: values a group (32, 64, 128) */
  uint8_t bits;              /* affine only: 4 or 8 bits a code */
  uint8_t scale_type;        /* affine only: 1 F16, 2 BF16, 3 F32; | 0x80 with zero points */
} llmp_decode_operand;
int llmp_hip_decode_vector(int decoder, const llmp_decode_operand* weight, uint64_t first, uint64_t outputs,
                           const float* x, uint64_t rows, uint64_t x_stride, float* y, uint64_t y_stride, void* stream);
/* RunVectorGlu of src/kernels/decode/products.h:120-139: y[t][j] = glu(gate row gate_first + j . x[t],
 * up row up_first + j . x[t]), each with its weight's tensor scale; one weight may be both (a
 * stacked gate and up). `glu` is ir::GluKind (src/ir/op.h:455): 0 SwiGLU, 1 GeGLU (erf), 2 GeGLU
 * (tanh), 3 SwiGLU with gate <= limit and |up| <= limit (src/kernels/decode/templates.cuh:73-90). The two weights share K;
 * their decoders are the same, or one of the six mixed pairs the reference instantiates
 * (src/kernels/decode/implementations.cc:73-81: an MXFP8, NVFP4, MXFP4 or affine split gate with a BF16 up, an NVFP4
 * or MXFP4 split gate with a Q8_0 up); any other pair is refused, as there. */
int llmp_hip_decode_vector_glu(int gate_decoder, const llmp_decode_operand* gate, uint64_t gate_first, int up_decoder,
                               const llmp_decode_operand* up, uint64_t up_first, uint64_t outputs, int glu, float limit,
                               const float* x, uint64_t rows, uint64_t x_stride, float* y, uint64_t y_stride,
                               void* stream);

/* RunRows of src/kernels/decode/products.h:172-183: out[i][:] = W[ids[i]][:] as F32 (times the row's tensor
 * scale) for i < count; ids are device I32; an id outside the matrix writes zeros and sets *bad (a device
 * I32, or null) to 1. Output rows 16-byte aligned, out_stride (floats) a multiple of 4. */
int llmp_hip_decode_rows(int decoder, const llmp_decode_operand* weight, const int32_t* ids, uint64_t count, float* out,
                         uint64_t out_stride, int32_t* bad, void* stream);

/* RunGrouped of src/kernels/decode/products.h:141-170: for each expert e its pairs p in [offsets[e],
 * offsets[e + 1]) compute y[pair_out[p] (or p)][j] = sum_k W_e[first + j][k] x[pair_rows[p]][k]. `experts` is a
 * device array of experts_count operands (any base address each) of the format's decoder, K (`k`) and N
 * (`n`); offsets (experts_count + 1), pair_rows and pair_out (or null) are device I32 arrays. The device skips
 * an expert whose operand's K or N is not the format's, a pair past `pairs`, and one naming a row past x_rows or
 * y_rows (its output row is left untouched). One launch; `rows_hint` (the reference's tile choice) is unused. */
int llmp_hip_decode_grouped(int decoder, const llmp_decode_operand* experts, uint64_t experts_count, uint32_t k, uint32_t n,
                            uint64_t first, uint64_t outputs, const int32_t* offsets, const int32_t* pair_rows,
                            const int32_t* pair_out, uint64_t pairs, const float* x, uint64_t x_rows, uint64_t x_stride,
                            float* y, uint64_t y_rows, uint64_t y_stride, uint64_t rows_hint, void* stream);

/* RunMatrix of src/kernels/decode/products.h:111-118: the same product for 1 to 65535 * 64 input rows on the
 * matrix cores (`path` 0, MatrixPath::kMma): the decoded weights and the inputs are rounded to the
 * decoder's matrix element (F16 for F16 and Q8_0 weights, BF16 for the others: products.h:27-33) and
 * summed in F32. `path` 1 (kFma, for devices without matrix instructions) is refused. One launch. */
int llmp_hip_decode_matrix(int decoder, const llmp_decode_operand* weight, uint64_t first, uint64_t outputs, const float* x,
                           uint64_t rows, uint64_t x_stride, float* y, uint64_t y_stride, int path, void* stream);

/* ------------------------------------------------------------ a yardstick
 * No counterpart in the reference: a launch that only reads `bytes` (whole 16-byte chunks at a 16-byte boundary),
 * eight loads in flight a lane, folded into `sink` (llmp_hip_stream_read_sink(cus) bytes, the caller's). What it
 * takes is what the launch latency and the memory system leave of the HBM peak at that size: the benchmark prints
 * it beside each streaming kernel's time. */
size_t llmp_hip_stream_read_sink(int compute_units);
int llmp_hip_stream_read(const void* data, size_t bytes, void* sink, int compute_units, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* LLMP_HIP_H_ */
