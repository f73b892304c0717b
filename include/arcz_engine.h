/*
 * arcz_engine.h -- the C ABI of the matmul dispatch: what the reference's Engine (zero/engine.h) offers for this
 * path, callable from any language.  The C++ class behind it (arcinferzero_amd/csrc/engine_hip.h) keeps the
 * reference's method names and argument meaning; a C++ caller can use that class directly.
 *
 * Every call returns 0 or a negative status; arcz_engine_error() gives the message of the last failure (the C++
 * methods throw std::runtime_error / std::logic_error as the reference's do; the exceptions stop here).
 * One engine per process is the expected use; all engines share the one stream of arcz_hip.h.
 */
#ifndef ARCZ_ENGINE_H
#define ARCZ_ENGINE_H
#include "arcz_hip.h"
#include "arcz_gguf.h"
#ifdef __cplusplus
extern "C" {
#endif

#define ARCZ_E_ENGINE (-100) /* an exception of the dispatch code: bad shapes, unsupported type, unloaded weight */

typedef struct arcz_engine arcz_engine;
typedef struct arcz_weight arcz_weight;       /* GpuWeight (zero/engine.h:27-34) */
typedef struct arcz_moe_layer arcz_moe_layer; /* the expert tensors of one layer (zero/engine_stream.h:285-306) */

const char* arcz_engine_error(void);

/* Engine::Engine + alloc_buffers (zero/engine.h:268, zero/engine_alloc.h:4-41): activation buffers for chunks of up
 * to max_chunk token rows of up to max_k values (aq int8 [M][K], asc f32 [K/32][M], absum int16 [K/16][M]). */
arcz_engine* arcz_engine_create(int max_chunk, int max_k);
/* Frees the engine's buffers -- except those that a live recorded launch list still names (arcz_mem_listed): these stay
 * allocated until the process ends, so that the list never replays on freed memory.  Free lists before their engine. */
void arcz_engine_destroy(arcz_engine* e);

/* make_weight + upload_padded (zero/engine_load.h:84-130, 157-196): N rows of K values as GGUF blocks of `type`
 * (2 = Q4_0, 8 = Q8_0, 11 = Q3_K, 12 = Q4_K, 13 = Q5_K, 14 = Q6_K, 18 = IQ3_XXS, 20 = IQ4_NL, 21 = IQ3_S, 23 = IQ4_XS,
 * 39 = MXFP4),
 * regrouped into the device layout -- every type in its own form, the GGUF byte count -- and uploaded.  Two more types,
 * 42 = Q2_0 (K a multiple of 64) and 0x41523447 = AR4_128 (K a multiple of 128), are taken as Q4_0: written out as Q4_0
 * blocks of the same values first (arcz_relayout_q4_0), so on the device they take Q4_0's bytes, not the file's. */
arcz_weight* arcz_weight_upload(arcz_engine* e, uint32_t type, int N, int K, const void* gguf, size_t bytes);
/* The same from a tensor of an open GGUF file (upload of zero/engine_load.h:84-196): a matrix (dims K, N) or an expert
 * tensor (dims K, N, experts) of type Q4_0 / Q8_0 / Q3_K / Q4_K / Q5_K / Q6_K / IQ3_XXS / IQ4_NL / IQ3_S / IQ4_XS / MXFP4 (or Q2_0 / AR4_128, as above), by name;
 * NULL + arcz_engine_error() when it is missing, of another type or shape.  The MoE layer: its three expert tensors (gate and up [NE][F][E], down [NE][E][F]). */
arcz_weight* arcz_weight_upload_gguf(arcz_engine* e, const arcz_gguf* g, const char* name);
arcz_moe_layer* arcz_moe_layer_upload_gguf(arcz_engine* e, const arcz_gguf* g, const char* gate, const char* up,
                                           const char* down, int NU);
int arcz_weight_free(arcz_engine* e, arcz_weight* w);
arcz_mem* arcz_weight_raw(const arcz_weight* w);
/* The row length the matmuls see: K, or -- Q8_0, Q4_0, IQ4_NL, MXFP4 rows of a K that is a multiple of 32 but not of
 * 256 -- K rounded up to whole superblocks, the rows having been padded with zero blocks as the reference's loader
 * pads them (zero/engine_load.h:371-387, src/quants.h:661-671).  The activations of such a matmul are rows of that
 * length whose tail is zero. */
int arcz_weight_k(const arcz_weight* w);
/* Marks w as the output head of a model with final-logit soft-capping (the reference's lm_head_ with hp.softcap,
 * zero/engine.h:984-990; kernel epilogue -DSOFTCAP=c, zero/kernels/decode.cl:882-886): arcz_engine_matmul over 1-8
 * tokens writes c * tanh(v / c) (then adds C when accumulating); with two-pass inputs both passes run without the cap
 * and the sum is capped (zero/engine.h:1081-1110).  Chunks of more than 8 tokens are not capped (the reference's heads
 * never see them).  cap = 0: no cap. */
int arcz_weight_set_softcap(arcz_weight* w, float cap);

/* The activation quantizer as a step of its own (quant_store16 of zero/kernels/ops.cl:38-72 inside the launch of
 * zero/engine.h:1256-1267): rows [0, T) of x (f32, row stride ldx) -> the engine's aq / asc / absum laid out for
 * Mp rows; rows [T, Mp) are zero.  The next matmul takes its form from T: 1 GEMV, 2..8 multi-token GEMV, else GEMM.
 * act32 = 1: one scale per 32 values, asc [K/32][Mp]; act32 = 0: one per 256 (the maximum over the superblock), asc
 * [K/256][Mp] (one-pass engines only).  The matmuls of that chunk take the same act32. */
int arcz_engine_quantize(arcz_engine* e, arcz_mem* x, int ldx, int K, int Mp, int T, int act32);
/* The fused producers (Engine::rmsnorm_quant, zero/engine.h:1256-1267, kernel zero/kernels/ops.cl:107-141; swiglu_quant,
 * zero/kernels/ops.cl:271-315 launched by run_rows_quant, zero/engine.h:1404-1440): rows [row_off, row_off + T) of x
 * through RMS norm with weight w (eps), or rows [gate(F) | up(F)] of gu through silu(gate) * up (gelu: the tanh form of
 * GELU; fused: rows of F finished values), quantized into the engine's activation buffers for Mp rows; they set the
 * form of the next matmul like arcz_engine_quantize.  hout (may be NULL): the normalized rows as f32, [Mp][K]. */
int arcz_engine_rmsnorm_quant(arcz_engine* e, arcz_mem* x, int row_off, arcz_mem* w, int K, int Mp, int T, int act32,
                              float eps, arcz_mem* hout);
int arcz_engine_swiglu_quant(arcz_engine* e, arcz_mem* gu, int F, int Mp, int T, int act32, int fused, int gelu);
/* Engine::add_norm_quant (zero/engine.h:1393-1403, kernel zero/kernels/ops_attn_g.cl:616-667): rows [0, T) of x become
 * (x + rmsnorm(t) * w) * s in place, and the next matmul's input is made from the new rows: rmsnorm(x) * w2 (norm2) or x
 * itself, quantized into the engine's activation buffers for Mp rows.  x, t: [T][K] f32; w, w2: [K] f32 (w2 may be NULL
 * without norm2). */
int arcz_engine_add_norm_quant(arcz_engine* e, arcz_mem* x, arcz_mem* t, arcz_mem* w, int K, int T, int Mp, float s,
                               arcz_mem* w2, int norm2, int act32, float eps);
/* Two-pass matmul inputs on or off (zero/engine.h:1034-1075 q2_init, 1080-1101 matmul; zero/kernels/ops.cl:49-59,
 * 73-101): every quantizing call above also stores what its int8 values miss, quantized the same way, in the second
 * half of the (re-allocated, twice as large) activation buffers, and every arcz_engine_matmul runs a second pass over
 * that half, accumulating into the first one's output (accumulate mode 2 is refused, as in the reference).  The
 * mixture-of-experts layer takes the first half only.  For 1-4 tokens the GEMV takes both halves in one launch, over
 * one read of the weights (zero/engine.h:1086-1088), with the result two launches give bit for bit (except one token of
 * Q4_K / Q5_K, whose one-token kernel groups a term's factors differently: equal to rounding); on = 2 keeps the two
 * launches at every token count.  Forgets the current chunk. */
int arcz_engine_two_pass(arcz_engine* e, int on);
/* The second halves (0 = int8 values, 1 = scales, 2 = 16-sums) as views, NULL in one-pass mode. */
arcz_mem* arcz_engine_residual(arcz_engine* e, int which);
/* Activations quantized by the caller, as the reference's benches do (bench/gemv_bench.cpp:103-129).  One-pass engines
 * only. */
int arcz_engine_set_activations(arcz_engine* e, const int8_t* aq, const float* asc, const int16_t* absum, int K, int Mp,
                                int T);
/* The engine's activation buffers (Engine::aq_, asc_, absum_; zero/engine_sessions.h:571). */
arcz_mem* arcz_engine_aq(arcz_engine* e);
arcz_mem* arcz_engine_asc(arcz_engine* e);
arcz_mem* arcz_engine_absum(arcz_engine* e);

/* Engine::matmul(name, w, Mp, C, ldc, c_off, acc, act32) (zero/engine.h:1080): C[:, c_off : c_off + N] (+)= act W^T
 * for the current chunk.  acc 0 = store, 1 = add to C, 2 = C = silu(C) * result (GEMM form only).  act32 must be what
 * the chunk was quantized with (an error otherwise); with act32 = 0 the superblock's scale stands for each of its
 * eight blocks (the reference's non-ACT32 kernels, zero/kernels/gemm.cl:489-520): the engine spreads it over a
 * per-32 scale array of its own in one small launch and runs the same kernels.  The fused gate + up GEMV and the
 * mixture-of-experts layer take per-32 chunks only. */
int arcz_engine_matmul(arcz_engine* e, const char* name, arcz_weight* w, int Mp, arcz_mem* C, int ldc, int c_off, int acc,
                       int act32);

/* Engine::gemv_gu(g, u, Mp, C) (zero/engine.h:1124-1146): one token, the FFN's gate and up matrices (same type, N = F
 * rows, K) in one launch -- rows [0, F) of gate at C[0, F), rows [0, F) of up at C[F, 2 F), each bit for bit what its
 * own arcz_engine_matmul gives.  1 = done; 0 = not taken, nothing was launched and the caller runs the two matmuls
 * (more than one token in the chunk, two-pass inputs, matrices of different type or shape, rows the LDS-staged GEMV
 * does not take); negative: an error. */
int arcz_engine_gemv_gu(arcz_engine* e, arcz_weight* g, arcz_weight* u, int Mp, arcz_mem* C);

/* arcz_engine_matmul for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments, same kernels, the same
 * result bit for bit; the one buffer a matmul uses beyond its inputs and outputs -- the workspace of partial tiles of
 * the short-chunk GEMM -- is the library's static device array (ARCZ_NOALLOC_SCRATCH_BYTES per GPU, held until the
 * process ends, its address taken once in arcz_init) instead of the engine's own buffer.  The call makes no hipMalloc,
 * hipFree or event; a launch whose partial tiles would not fit the array is refused with ARCZ_E_ENGINE and a message
 * that names both sizes; launches are not timed by the engine's profile.  Every call on a GPU shares that GPU's array
 * and finds the last call's contents in it (the kernels write every partial tile before reading it: nothing needs
 * clearing): calls that overlap in time on one GPU race. */
#define ARCZ_NOALLOC_SCRATCH_BYTES (32u << 20)
int arcz_engine_matmul_noalloc(arcz_engine* e, const char* name, arcz_weight* w, int Mp, arcz_mem* C, int ldc, int c_off,
                               int acc, int act32);

/* Expert tensors of one MoE layer: gate, up [NE][F][E] and down [NE][E][F] as GGUF blocks of `type`, with the bytes the
 * caller holds of each: a tensor whose byte count is not what its type and shape come to (rows x K / block x block
 * bytes) is refused before anything is read (NULL + arcz_engine_error()). */
arcz_moe_layer* arcz_moe_layer_upload(arcz_engine* e, uint32_t type, const void* gate, size_t gate_bytes, const void* up,
                                      size_t up_bytes, const void* down, size_t down_bytes, int NE, int NU, int E, int F);
/* Engine::layer_moe (zero/engine_moe.h:8-361, standard experts, no shared expert): x[t] += sum_k w_k expert_k(h[t]) for
 * the T tokens whose quantized h is the current activation chunk; logits: router logits [T][ldl] f32. */
/* The hidden and FFN widths the layer works with: E and F, or -- where they are not whole superblocks (multiples of
 * 256) -- E and F rounded up, the tensors having been padded with zero rows and zero blocks as the reference's loader
 * pads them (zero/engine_load.h:371-387; columns: Q8_0, Q4_0, IQ4_NL and MXFP4 only).  The activations and the rows of
 * x are then that wide, their tails zero. */
int arcz_moe_layer_dims(const arcz_moe_layer* L, int* E, int* F);
int arcz_engine_layer_moe(arcz_engine* e, arcz_moe_layer* L, arcz_mem* logits, int ldl, arcz_mem* x, int T, int Mp);
/* The same with the shared expert's term (moe_combine's sgate * sh, zero/kernels/moe.cl:344-352): sh [T][E] f32 is the
 * shared expert's output for the chunk (computed by the caller with arcz_engine_matmul, as zero/engine_moe.h:66-84
 * does); x[t] += sgate[t] * sh[t] + the experts' sum, sgate[t] = sigmoid(logits[t][NE]) for rows of ldl > NE values. */
int arcz_engine_layer_moe_sh(arcz_engine* e, arcz_moe_layer* L, arcz_mem* logits, int ldl, arcz_mem* x, int T, int Mp,
                             arcz_mem* sh);
/* The reference's routing variants (zero/kernels/moe.cl:17-46, set by zero/engine_moe.h:99-116): escale [NE] (host f32,
 * its -DESCALE: each chosen expert's weight times its scale, after the normalization) or ebias [NE] + rscale (its
 * -DROUTE_DS -DRSCALE: scores sqrt(softplus(logit)), experts chosen by score + bias, weights score / (sum + 1e-20) *
 * rscale, shared-expert gate 1).  Both NULL: the softmax routing again.  Not both at once. */
int arcz_moe_layer_set_routing(arcz_engine* e, arcz_moe_layer* L, const float* escale, const float* ebias, float rscale);
/* Frees a layer's expert tensors and routing tables. */
int arcz_moe_layer_free(arcz_engine* e, arcz_moe_layer* L);
/* sgate [max_chunk] f32: the shared expert's gate per token, as the last routing wrote it. */
arcz_mem* arcz_engine_moe_sgate(arcz_engine* e);
/* The routing step alone (moe_route + moe_scan + moe_scatter, zero/engine_moe.h:111-133) with tiles of tm slots, and
 * its buffers: which = 0 ids, 1 wts, 2 offs, 3 tiles, 4 tstart, 5 stok, 6 swt, 7 inv, 8 h (f32), 9 hq, 10 hsc, 11 y,
 * 12 hbs (int16 sums of each 16 values of hq, [F/16][slots]). */
int arcz_engine_moe_route(arcz_engine* e, arcz_moe_layer* L, arcz_mem* logits, int ldl, int T, int tm);
arcz_mem* arcz_engine_moe_buffer(arcz_engine* e, int which);
int arcz_engine_moe_slots(arcz_engine* e);

/* The start-up check of the tuned GEMMs against the simple one on the reference's LCG data, both against integer sums
 * counted on the host (the pattern of xmx_check, zero/engine_setup.h:424-520): every weight type, the three accumulate
 * modes, K in one piece and in several.  0, or ARCZ_E_ENGINE with the first
 * difference in arcz_engine_error(). */
int arcz_engine_self_check(void);

/* Engine::profile / collect_profile (zero/engine.h:936-950): per-launch device time summed by name. */
void arcz_engine_profile(arcz_engine* e, int on);
int arcz_engine_profile_collect(arcz_engine* e);
int arcz_engine_profile_get(arcz_engine* e, const char* name, double* ms, int* launches);
/* Minimum and median of the collected per-launch times of `name` (the reference's benches print median and minimum,
 * bench/gemv_bench.cpp:215-229). */
int arcz_engine_profile_stats(arcz_engine* e, const char* name, double* min_ms, double* median_ms);
void arcz_engine_profile_reset(arcz_engine* e);
uint64_t arcz_engine_rd_bytes(arcz_engine* e);

/* Host helpers (no GPU): byte counts, the GGUF -> device planes regrouping, quantizers and seeded generators. */
size_t arcz_gguf_bytes(uint32_t type, size_t rows, int K);
size_t arcz_planes_bytes(uint32_t type, size_t rows, int K);
int arcz_repack_planes(uint32_t type, size_t rows, int K, const uint8_t* gguf, uint8_t* planes);
/* AR4_128 (0x41523447) and Q2_0 (42) rows (src/quants.h:531-542, 607-616) written out as Q4_0 blocks with the same
 * values (d * (q - 8) with the 128-block's d; d * ((q + 7) - 8)): what make_weight does with these two types before
 * anything else.  K in whole source blocks (128, 64); dst: rows * K / 32 * 18 bytes, or NULL to ask for the count only.
 * Returns the source bytes (rows * K / 128 * 66, rows * K / 64 * 18), 0 for another type or a K that does not fit. */
size_t arcz_relayout_q4_0(uint32_t type, size_t rows, int K, const uint8_t* src, uint8_t* dst);
/* The IQ3_S codebook (ggml's iq3s_grid, src/iq_tables.h:297) as the kernels take it in their `tabs` argument: 512 words,
 * byte j of a word = magnitude j of the entry (1, 3, ..., 15). */
void arcz_iq3s_grid(uint32_t* out512);
/* ... and IQ3_XXS's: 256 words (ggml's iq3xxs_grid, the reference's src/iq_tables.h). */
void arcz_iq3xxs_grid(uint32_t* out256);
/* quantize_rows_q8_0 (src/quants.h:429-442) and this library's own Q4_K / Q5_K / Q6_K / IQ4_XS / IQ3_S / IQ4_NL / MXFP4 block makers (input generators). */
int arcz_quantize_rows(uint32_t type, const float* src, size_t N, int K, uint8_t* out);
void arcz_gen_normal(uint64_t seed, size_t n, float mean, float std, float* out);
int arcz_gen_weights(uint32_t type, uint64_t seed, size_t N, int K, float std, uint8_t* out);

#ifdef __cplusplus
}
#endif
#endif
