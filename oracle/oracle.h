/*
 * CPU oracle for the quantized linear-layer path: TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the reference's CPU definitions of the path
 * (src/kernels/reference/{decode.cc,decode_exl3.cc,exec.cc} and the scalar
 * block references of tests/unit/dsv4_fast_test.cc). It is the checker the
 * parity tests compare the HIP kernels against and the timed CPU baseline of
 * the benchmark. Nothing in the shipped library calls it.
 *
 * Parity pins (tests/test_oracle_*.py): element conversions against numpy's
 * IEEE float16 and closed forms; EXL3 codebooks against the 18 golden vectors
 * of tests/unit/reference_decode_test.cc:677-682; tile placement against that
 * test's independent derivation (:699-747); Hadamard rows against an explicit
 * Hadamard-matrix product (:754-814); Q4_K/Q8_0 block sums against numpy
 * brute force; the MXFP8 quantizer against the invariants of
 * tests/unit/qwen38_fast_test.cc:179-218; router and grouping against numpy
 * stable sorts.
 *
 * parity unpinned: orc_q8_1_quantize's rounding flavour (x / d against x * (1/d))
 * and its fp16 sum field `s`. The reference takes both from ggml, which is not
 * in the reference tree; no in-tree fixture fixes them. Flavor 0 here is the
 * device definition (IEEE divide, butterfly-ordered sum), flavor 1 the ggml CPU
 * definition (multiply by the reciprocal, s = d * sum(q)).
 * parity unpinned as well: Q6_K's and Q5_K's bit layouts (ggml's dequantize_row_q6_K, _q5_K restated; no vector in the
 * reference), pinned only against numpy's reading of the same published layout; the IQ4_NL codebook (ggml's kvalues_iq4nl, restated from llama.cpp's
 * ggml-common.h; the reference reads it from ggml and holds no vector for the type). Its layout and
 * arithmetic are pinned against numpy and a hand-built block.
 */
#ifndef LLMP_ORACLE_H_
#define LLMP_ORACLE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- element conversions: src/kernels/reference/decode.cc:341-428 ---- */
float orc_f16_to_f32(uint16_t bits);
uint16_t orc_f32_to_f16(float value);
float orc_bf16_to_f32(uint16_t bits);
uint16_t orc_f32_to_bf16(float value);
float orc_e4m3_to_f32(uint8_t bits);
float orc_e8m0_to_f32(uint8_t bits);
float orc_e2m1_to_f32(uint8_t code); /* decode.cc:424-428 */
/* Saturating-finite round-to-nearest-even E4M3, what __nv_cvt_float2_to_fp8x2(
 * ..., __NV_SATFINITE, __NV_E4M3) gives (src/kernels/ggml/mxfp8_quant.cuh:38-46). */
uint8_t orc_f32_to_e4m3(float value);

/* ---- Q8_1 activations: src/ir/op.h:400-405, src/kernels/ggml/llmp_moe.cu:521-536,
 * src/kernels/ggml/kv_quant.cuh:27-43, src/kernels/ggml/llmp_ops.cc:2568-2576 ---- */
enum { ORC_Q8_DEVICE = 0, ORC_Q8_GGML_CPU = 1 };
/* One row of k floats into padded_k / 32 blocks of 36 bytes {f16 d; f16 s; i8 qs[32]};
 * the blocks past k are zero. */
void orc_q8_1_quantize_row(const float* x, int64_t k, int64_t padded_k, uint8_t* out, int flavor);
/* d * q of each block: src/kernels/reference/decode.cc:158-170. */
void orc_q8_1_decode_row(const uint8_t* blocks, int64_t k, float* y);

/* ---- KV cache store: src/kernels/ggml/kv_quant.cuh:27-69 (GGML's reference Q8_0 and Q4_0
 * quantizers step by step, every operation an IEEE one). One row of k floats into k / 32 blocks
 * of 34 (ORC_TYPE_Q8_0) or 18 (ORC_TYPE_Q4_0) bytes. ---- */
void orc_kv_quantize_row(int type, const float* x, int64_t k, uint8_t* out);

/* ---- weight blocks: src/format/encoding.cc:110-116 ---- */
enum { ORC_TYPE_Q4_0 = 2, ORC_TYPE_Q4_1 = 3, ORC_TYPE_Q5_0 = 6, ORC_TYPE_Q5_1 = 7, ORC_TYPE_Q8_0 = 8, ORC_TYPE_Q4_K = 12, ORC_TYPE_MXFP4 = 39, ORC_TYPE_IQ4_NL = 20, ORC_TYPE_Q5_K = 13, ORC_TYPE_Q6_K = 14 }; /* ggml_type values */
int orc_block_bytes(int type);    /* 18 / 20 / 22 / 24 / 34 / 144, MXFP4 17, IQ4_NL 18, Q5_K 176, Q6_K 210 */
int orc_block_elements(int type); /* 32, the K-quants 256 */
/* The Q4_K 6-bit scale and minimum of sub-block g: tests/unit/dsv4_fast_test.cc:180-183. */
void orc_q4_k_scale_min(const uint8_t* scales12, int g, int* scale, int* minimum);
/* Decode rows of blocks to floats (the ggml dequantization of those bytes). */
void orc_decode_row(int type, const uint8_t* row, int64_t k, float* y);
/* Per-block int32 sums over identical Q8_1 bytes. Q8_0 and the legacy 4/5-bit blocks:
 * sums[0] = sum w*q (code*q) of the 32 values (src/kernels/ggml/vecq.cu:398-418,
 * tests/unit/dsv4_fast_test.cc:154-158). Q4_K: sums[0..7] = sum code*q per
 * sub-block, sums[8..15] = sum q per sub-block (tests/unit/dsv4_fast_test.cc:185-191).
 * MXFP4: sums[0] = sum of twice the E2M1 values times q (vecq.cu:421-435, the values of
 * src/kernels/reference/decode.cc:424-428). */
void orc_block_sums(int type, const uint8_t* wblock, const uint8_t* q8, int32_t* sums);
/* One weight block times its Q8_1 blocks in double. */
double orc_block_product(int type, const uint8_t* wblock, const uint8_t* q8);

/* ---- decode products: src/kernels/decode/products.h:96-109 over the operand of
 * src/kernels/decode/operand.h:74-97, values as src/kernels/reference/decode.cc decodes them ---- */
enum {
  ORC_DECODER_BF16_DENSE = 0, ORC_DECODER_F16_DENSE, ORC_DECODER_Q8_0_BLOCKS, ORC_DECODER_NVFP4_SPLIT,
  ORC_DECODER_NVFP4_ATOMS, ORC_DECODER_NVFP4_INTERLEAVED, ORC_DECODER_NVFP4_GGML_BLOCKS, ORC_DECODER_MXFP8_SPLIT,
  ORC_DECODER_MXFP8_ATOMS, ORC_DECODER_MXFP4_SPLIT, ORC_DECODER_MXFP4_ATOMS, ORC_DECODER_AFFINE_SPLIT
}; /* operand.h:26-41 */
typedef struct orc_decode_operand { /* operand.h:74-97, field for field */
  const uint8_t* data;
  const uint8_t* scales;
  const float* tensor_scale;
  const uint8_t* biases;
  uint32_t k, rows, rows_per_scale, pad;
  uint64_t row_bytes;
  uint32_t scale_row_bytes;
  uint16_t group;
  uint8_t bits, scale_type;
} orc_decode_operand;
float orc_ue4m3_to_f32(uint8_t bits); /* decode.cc:407-411: E4M3's value up to 0x7E, NaN from 0x7F */
/* Value j of row `row`, before the tensor scale. */
float orc_decode_value(int decoder, const orc_decode_operand* w, uint64_t row, uint64_t j);
/* y[t][j] = tensor_scale(first + j) * sum_k W[first + j][k] x[t][k] in double; 1 for an unknown decoder. */
int orc_decode_vector(int decoder, const orc_decode_operand* w, uint64_t first, uint64_t outputs, const float* x,
                      uint64_t rows, uint64_t x_stride, float* y, uint64_t y_stride, int threads);

/* RunVectorGlu, products.h:120-139: y[t][j] = glu(gate row . x[t], up row . x[t]); glu is ir::GluKind
 * (src/ir/op.h:455), the functions those of src/kernels/reference/exec.cc:248-262. */
int orc_decode_vector_glu(int decoder, const orc_decode_operand* gate, uint64_t gate_first, int up_decoder,
                          const orc_decode_operand* up, uint64_t up_first, uint64_t outputs, int glu, float limit,
                          const float* x, uint64_t rows, uint64_t x_stride, float* y, uint64_t y_stride, int threads);

/* RunMatrix's tensor-core path, products.h:27-33 and 111-118: weights and inputs rounded to the decoder's
 * matrix element (F16 for F16 and Q8_0 weights, BF16 otherwise), double sums here. */
int orc_decode_matrix(int decoder, const orc_decode_operand* w, uint64_t first, uint64_t outputs, const float* x,
                      uint64_t rows, uint64_t x_stride, float* y, uint64_t y_stride, int threads);
/* RunGrouped, products.h:141-170: an expert worklist's products; experts whose K or N differ, pairs past
 * `pairs` and pairs naming rows past x_rows or y_rows are skipped. */
int orc_decode_grouped(int decoder, const orc_decode_operand* experts, uint64_t experts_count, uint32_t k, uint32_t n,
                       uint64_t first, uint64_t outputs, const int32_t* offsets, const int32_t* pair_rows,
                       const int32_t* pair_out, uint64_t pairs, const float* x, uint64_t x_rows, uint64_t x_stride, float* y,
                       uint64_t y_rows, uint64_t y_stride);

/* ---- GLU: src/kernels/reference/exec.cc:206-214,248-262 ---- */
enum { ORC_GLU_NONE = 0, ORC_GLU_SWIGLU = 1, ORC_GLU_SWIGLU_CLAMP = 2, ORC_GLU_GEGLU = 3 };
double orc_glu(int kind, double gate, double up, double limit);

/* ---- llmp.vecq on the CPU: the VecQDesc of src/kernels/ggml/vecq.h:22-41 ---- */
typedef struct {
  const void* w;
  const void* g;
  const void* y;
  const int32_t* ids;
  float* dst;
  int ncols_x, nrows, stride_row, stride_expert, y_token, y_slot, ids_stride;
  int used, tokens, dst_token, dst_slot, glu;
  float limit;
} orc_vecq_desc;
/* Every (token, slot, row) in double over the Q8_1 bytes, rounded once to float.
 * Returns 0, or 1 for an id outside [0, experts) (exec.cc:978-981) when experts > 0.
 * threads > 1 splits the rows over OpenMP threads. */
int orc_vecq(int type, const orc_vecq_desc* d, int experts, int threads);
/* The int32 sums of every (row, block) of a dense one-token product:
 * out[(row * blocks + b) * per + i], per = 1 (Q8_0) or 16 (Q4_K). */
void orc_vecq_block_sums(int type, const void* w, const void* y, int k, int nrows, int stride_row,
                         int32_t* out);

/* ---- MXFP8: src/kernels/ggml/mxfp8_quant.cuh:19-46, mxfp8_cutlass.h:26-57,
 * src/format/layout.h:96-113 ---- */
uint32_t orc_mxfp8_scale_code(float amax);
float orc_mxfp8_inverse_scale(uint32_t e);
uint64_t orc_scale_atom_offset(uint64_t row, uint64_t block, uint64_t blocks);
/* rows of k floats -> codes [rows][k] and swizzled scales for the rows rounded up to 128
 * (padding rows zero): src/kernels/ggml/llmp_ops.cu:610-648. */
void orc_mxfp8_quantize(const float* x, int64_t x_stride, int64_t k, int64_t rows, uint8_t* codes,
                        uint8_t* scales);
/* [n][k/32] scales -> atoms: src/kernels/ggml/llmp_ops.cu:652-663. */
void orc_mxfp8_swizzle(const uint8_t* in, int64_t n, int64_t blocks, uint8_t* out);
/* One element of D = A * B^T from codes and swizzled scales, in double:
 * src/kernels/ggml/mxfp8_cutlass.h:12-24. */
double orc_mxfp8_dot(const uint8_t* a_codes, const uint8_t* a_scales, int64_t row_a,
                     const uint8_t* b_codes, const uint8_t* b_scales, int64_t row_b, int64_t k);
/* Whole product with float accumulation per 32-block order, out float [m][n]. */
void orc_mxfp8_gemm(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                    const uint8_t* b_scales, int64_t m, int64_t n, int64_t k, float* d, int threads);
/* Weight vector product: y = sum_blocks (sum_32 E4M3(code) * x) * 2^(s-127) with split scales:
 * src/kernels/ggml/llmp_ops.cu:145-224. */
void orc_mxfp8_gemv(const uint8_t* codes, const uint8_t* scales, int64_t n, int64_t k,
                    const float* x, int64_t tokens, float* y);

/* ---- MoE: src/kernels/reference/exec.cc:279-315,1003-1025,1728-1856 ---- */
/* softmax, top-`used` (ties to the lower index, NaN last), weights over max(sum, 2^-14) * scale. */
void orc_route(const float* logits, int64_t experts, int64_t used, int64_t tokens, int normalize,
               float scale, int32_t* ids, float* weights);
/* order[i] = pair index t*U+u in expert order; offsets[experts + 1]. Returns 1 on a bad id. */
int orc_expert_sort(const int32_t* ids, int64_t pairs, int64_t experts, int32_t* order,
                    int32_t* offsets);
/* out[:, t] = sum_u x[:, u, t] * w[u, t] in slot order, float arithmetic as
 * src/kernels/ggml/llmp_fused.cu:200-240 without scales or a shared expert. */
void orc_expert_reduce(const float* x, const float* w, int64_t width, int64_t used, int64_t tokens,
                       float* out);

/* ---- EXL3: src/kernels/reference/decode_exl3.cc ---- */
enum { ORC_CB_3INST = 0, ORC_CB_MCG = 1, ORC_CB_MUL1 = 2 };
uint16_t orc_exl3_codebook(int codebook, uint16_t state);
uint16_t orc_exl3_state(const uint8_t* tile, uint32_t bits, uint32_t t);
/* position t of a tile -> row * 16 + column. */
void orc_exl3_placement(uint8_t* at256);
/* The rotated-basis weights, F16 bits [k][count] for columns [first, first + count). */
void orc_exl3_rotated(const uint8_t* trellis, int64_t k, int64_t n, int bits, int codebook,
                      int64_t first, int64_t count, uint16_t* out);
/* W rows [n][k] float for outputs [first, first + count): decode_exl3.cc:217-265. */
void orc_exl3_rows(const uint8_t* trellis, const uint16_t* suh, const uint16_t* svh, int64_t k,
                   int64_t n, int bits, int codebook, int64_t first, int64_t count, float* out);
/* The device path's definition of the linear (src/kernels/exl3/linear.h:4-31):
 * xh = f16(H(x * suh) / sqrt(128)); acc = xh * W^; y = H(acc) / sqrt(128) * svh, in double
 * but for xh's one rounding. x F16 [m][k], y float [m][n]. */
void orc_exl3_linear(const uint8_t* trellis, const uint16_t* suh, const uint16_t* svh, int64_t k,
                     int64_t n, int bits, int codebook, const uint16_t* x, int64_t m, float* y,
                     int threads);
/* Its two stages: the transformed input xh (F16 [m][k]), and the product and output transform
 * over a given xh. */
void orc_exl3_input(const uint16_t* suh, int64_t k, const uint16_t* x, int64_t m, uint16_t* xh);
void orc_exl3_product(const uint8_t* trellis, const uint16_t* svh, int64_t k, int64_t n, int bits,
                      int codebook, const uint16_t* xh, int64_t m, float* y, int threads);

/* Attention over a Q8_0 or Q4_0 KV cache decoded exactly, in double (exec.cc:1027-1085 of the reference); with
 * q8_1_q the query rows pass through Q8_1 first, as the device's K product takes them. Layouts in oracle.c. */
void orc_attention_quant(int type, const float* q, const uint8_t* k, const uint8_t* v, int64_t cell_stride,
                         int64_t head_stride, const uint16_t* mask, const float* sinks, int64_t d, int64_t heads,
                         int64_t kv_heads, int64_t rows, int64_t cells, float scale, float softcap, int q8_1_q,
                         float* out, int threads);

int orc_max_threads(void);

#ifdef __cplusplus
}
#endif

#endif /* LLMP_ORACLE_H_ */
