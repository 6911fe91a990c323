// TEST INFRASTRUCTURE — CPU oracle for the batched quantized decode path.
//
// This is a CPU restatement of the reference's arithmetic, used only as the checker by tests/, by the
// smoke check and by the cpu_baseline leg of the benchmark. Nothing in the product library links,
// loads or calls it.
//
// Pinning status of each function (what, other than this file, fixes its answers):
//   qwo_dq_row type 8 (Q8_0)  pinned: compared against the reference's own src/ggml_dq.c compiled
//                             into oracle/_ref (when that is built), against hand-made known answers,
//                             and against the closed form int8 * fp16.
//   qwo_dq_row types 12, 13, 14, 20, 23 (Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS) and 0, 1, 30 (float, binary16,
//                             bfloat16)  pinned: written per value position (the reference walks blocks with
//                             running pointers), compared bit for bit against the reference's src/ggml_dq.c
//                             in oracle/_ref on random blocks, against the committed values that library gave
//                             (tests/golden/dq_formats.npz) and against one hand block per format.
//   qwo_dq_row type 21 (IQ3_S) pinned by: hand-made known-answer blocks (all-ones, all-negative, scale
//                             31, high-bit codebook entry 256, denormal / largest fp16 scale), the
//                             codebook CRC-32 0xf576e4f3, the closed form +-d*(2s+1)*g, and agreement of
//                             the two formulations the reference carries (qwo_dq_row = per-32 decoder,
//                             qwo_dq_row_tab = 16-value units through the pre-signed table). Equivalence
//                             with upstream ggml's dequantize_row_iq3_s rests on the reference's Metal
//                             text (no upstream code or gguf package exists in this environment).
//   qwo_qmv_*                 pinned by float64 recomputation in numpy from dequantized rows and by
//                             linearity / row-independence properties.
//   qwo_select                pinned by a brute-force stable-argsort restatement in numpy, crafted ties,
//                             the closed-form softmax / sigmoid, and dedupe invariants.
//   qwo_moe_layer_*           pinned by a numpy float64 recomputation on small shapes.
//   qwo_moe_pack              pinned by counting-sort invariants (exclusive scan, permutation).
//   qwo_hyper_gg              pinned by: the cases the mathematics fixes (a zero mix_up matrix makes every gate
//                             sigmoid(0) = 1/2; zero inject sums make the residual coefficient exactly 1; scaling
//                             the streams leaves the normalised vector unchanged; one-hot mix_down / mix_up rows
//                             pick single terms), an element-by-element loop on a tiny shape, and a float64
//                             matrix statement in numpy. The reference holds no dump of this step (its
//                             tools/hc_ref.py reads files a model run writes).
#pragma once
#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

// ---- scalar helpers
float qwo_h2f(uint16_t h);   // IEEE binary16 -> binary32, exact
uint16_t qwo_f2h(float f);   // binary32 -> binary16, round to nearest even
float qwo_bf2f(uint16_t h);  // bfloat16 -> binary32, exact

// ---- block formats (reference: src/gguf.c:15-25): values per block / bytes per block, 0 if unsupported here
int qwo_block_values(int type);
int qwo_block_bytes(int type);
size_t qwo_row_bytes(int type, int K);

// ---- dequantisation. Same contract as the reference's qw_ggml_dq_row (src/ggml_dq.h:8): one row of K
// values, K a multiple of the block size; false when the type is not handled. Types: 0, 1, 30 (float, binary16,
// bfloat16), 8 (Q8_0), 12, 13, 14 (Q4_K, Q5_K, Q6_K), 20, 23 (IQ4_NL, IQ4_XS), 21 (IQ3_S).
bool qwo_dq_ok(int type);
bool qwo_dq_row(int type, const void *src, float *dst, int K);
// Second, independent formulation of the same values: 16-value units decoded through the pre-signed
// codebook table, then multiplied by the sub-block scale (reference: kernels/moe_gg.metal:321-334, 396-407).
bool qwo_dq_row_tab(int type, const void *src, float *dst, int K);
// The pre-signed table itself: 8192 entries of four binary16 values; entry (g | s << 9) holds the four
// magnitudes of codebook entry g with the sign of value j taken from bit j of s (kernels/moe_gg.metal:495-500).
void qwo_tab_iq3ss(uint16_t *tab /* [8192 * 4] */);
const uint32_t *qwo_iq3s_table(void); // the 512-entry codebook

// ---- dense matvec y[b][row] = sum_k W[row][k] * x[b][k] (reference: kernels/qmv_gg.metal:17-39).
// W: N rows of qwo_row_bytes(type, K); x: binary16 [nb][xstride]; y: [nb][ystride].
// _f32: weights to float, activation to float, float accumulation in index order (the CPU reference path).
// _f64: the same products accumulated in double (the tight numerical reference).
// threads <= 0 means all cores (OpenMP over rows).
void qwo_qmv_f32(int type, const uint8_t *W, int N, int K, const uint16_t *x, int nb, int xstride, float *y, int ystride,
                 int threads);
void qwo_qmv_f64(int type, const uint8_t *W, int N, int K, const uint16_t *x, int nb, int xstride, double *y, int ystride,
                 int threads);

// ---- router (reference: kernels/moe_gg.metal:25-41): logits[t][r], row stride E + 1; r == E is the
// shared-expert gate vector. wfmt: 1 = binary16 weights, 30 = bfloat16 weights. Accumulates in double,
// stores float (a summation-order-free target for any float implementation).
void qwo_router(int wfmt, const uint16_t *Wr, const uint16_t *Wsg, const uint16_t *x, int nb, int D, int E, float *logits);

// ---- expert selection + dedupe (reference: kernels/moe_gg.metal:110-189).
// Result layout for gnb token columns (8 = the reference's gg_sel, 16 = the wide layout), GU = gnb * topk:
//   uint32 U; uint32 ue[GU]; uint32 mask[GU]; uint8 slot[GU][gnb]; float w[gnb][topk + 1]
size_t qwo_sel_bytes(int gnb, int topk);
// Entries of ue / mask at index >= U and every unused slot byte are written as zero.
void qwo_select(const float *logits, int nbr, int E, int topk, int gnb, void *sel);
// Top-k ids alone: ids[t][k] by rank, ties to the lowest index (repeated argmax).
void qwo_topk(const float *logits, int nbr, int E, int topk, uint32_t *ids);

// ---- one MoE layer (reference: kernels/moe_gg.metal:428-483, 534-663; layer math kernels/moe_decode.metal:1-12).
typedef struct {
    int D, I, E, topk;
    int fgu, fd;             // ggml type of routed gate/up and routed down
    int fsg, fsu, fsd;       // ggml type of shared gate, up, down
    const uint8_t *Wg, *Wu;  // [E][I][row_bytes(fgu, D)]
    const uint8_t *Wd;       // [E][D][row_bytes(fd, I)]
    const uint8_t *Wsg, *Wsu; // [I][row_bytes(., D)]
    const uint8_t *Wsd;      // [D][row_bytes(fsd, I)]
} qwo_moe_weights;
// logits: [nb][E + 1] float (from qwo_router or from the device); x binary16 [nb][D].
// _f32 mirrors the reference kernels' precision: float dot products, H kept in float, rank-order combine,
// out rounded to binary16. _f64 does everything in double and returns double out[nb][D].
// Optional outputs (may be NULL): H [nb][topk+1][I], sel (qwo_sel_bytes(gnb, topk)).
void qwo_moe_layer_f32(const qwo_moe_weights *m, const float *logits, const uint16_t *x, int nb, int gnb, uint16_t *out,
                       float *H, void *sel, int threads);
void qwo_moe_layer_f64(const qwo_moe_weights *m, const float *logits, const uint16_t *x, int nb, double *out, int threads);

// ---- ragged packing for the grouped path (reference: kernels/moe_prefill.metal:15-93).
// ids: P = rows * topk expert ids in flat order. counts[E], offs[E] = exclusive scan, pos_of[P] = position of
// pair p in expert-sorted order (stable: earlier flat index first), tiles[max_tiles][4] = {expert,row0,row1,0}
// for row blocks of tm rows, unused tiles zeroed. Returns the number of tiles in use.
int qwo_moe_pack(const uint32_t *ids, int P, int E, int tm, uint32_t *counts, uint32_t *offs, uint32_t *pos_of,
                 uint32_t *tiles, int max_tiles);

// Hyper-connection of the GGUF profile (kernels/hyper_gg.metal:94-233; the reference's own float64 statement is
// tools/hc_ref.py:60-70), one call for NB tokens, everything in float64:
//   js[s]   = apply ? 2 sigmoid(sum_q inj[q][s] / HC) : 0            (kernels/hyper_gg.metal:47-51)
//   h1[s]   = h[s] + out * js[s]
//   r[s]    = 1 / sqrt(mean_j h1[s][j]^2 + 1e-6);  y[s][j] = h1[s][j] r[s] w[s D + j]
//   d       = Wd y (LR rows over the HC D columns);  sx = silu(d / HC);  u = Wu sx
//   x[j]    = mean_s sigmoid(u[s D + j]) y[s][j]
//   injo[s][q] = sum_j Wi[q][s D + j] y[s][j]                          (only when Wi is given)
// h1 is returned in h_out whether or not the residual was applied.
void qwo_hyper_gg(int D, int HC, int LR, int NB, int apply, const float *h, const uint16_t *out_f16, const float *inj, const float *w,
                  const uint16_t *Wd_bf16, const uint16_t *Wi_bf16, const uint16_t *Wu_bf16, double *h_out, double *x, double *inj_out);

int qwo_max_threads(void);

#ifdef __cplusplus
}
#endif
