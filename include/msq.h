/* libmsq: MI355X (gfx950) quantized matvec / MoE kernels over raw GGUF blocks -- C ABI.
 *
 * Drop-in boundary for the "quant" operator module of MacSeek (reference: src/kernels/quant.hpp). Every entry point
 * below names the reference function it replaces. Conventions carried over from the reference:
 *   - functions only ENQUEUE work on the given stream (reference: "only encode; never commit/wait", quant.hpp:3);
 *     `stream` is a hipStream_t passed as void* (NULL = the default stream). Dependent calls on one stream are
 *     ordered by the stream, so the reference's explicit Enc::barrier() between them has no counterpart.
 *   - weights are raw GGUF block rows: an [in -> out] matrix is rows = out rows of cols = in elements
 *     (quant.hpp:4); weight bases need 4-byte alignment only, activations / outputs 16-byte alignment
 *     (docs/modules/quant.md:27-30). Activations must be finite. One token (msq_matvec, msq_matvec_rmsnorm, gate/up of
 *     the one-token MoE layer) is F32-activation arithmetic like the reference's: the block formats multiply integer
 *     payloads with activations rounded at 2^-16 of the largest value of their run of 8 to 32 columns (no range limit),
 *     Q8_0 and the dense types keep fp32. Several tokens (msq_matvec_n from n = 2, the prefill paths) and the down
 *     projection of the MoE layer stage activations as fp16 pairs, as the reference does for its n > 1 paths: there
 *     |x| <= 65504 (larger values turn into infinities); MoE routing weights up to 5 keep the down projection's
 *     inputs inside that range.
 *   - all buffers are caller-owned device memory; MsqBuffer mirrors ms::Buffer {buf, off, size}
 *     (src/core/metal.hpp:11-18).
 *   - misuse is reported, not aborted: functions return 0 on success or a negative MSQ_ERR_* code and leave a
 *     message for msq_last_error(). The C++ shim (include/macseek_amd/quant.hpp) turns a non-zero status into the
 *     reference's behaviour: print "macseek quant: ... unsupported" and abort() (src/kernels/quant.mm:34-37).
 */
#ifndef MSQ_H
#define MSQ_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml type ids (reference: src/kernels/quant_types.hpp:9-11) */
enum {
  MSQ_T_F32 = 0, MSQ_T_F16 = 1, MSQ_T_Q8_0 = 8, MSQ_T_Q5_K = 13, MSQ_T_Q6_K = 14, MSQ_T_IQ2_XXS = 16,
  MSQ_T_IQ1_S = 19, MSQ_T_IQ4_NL = 20, MSQ_T_BF16 = 30
};

enum {
  MSQ_OK = 0,
  MSQ_ERR_UNSUPPORTED = -1, /* type / shape / combination the kernels do not cover (reference: die()) */
  MSQ_ERR_ARGUMENT = -2,    /* null buffer, size too small, count out of range */
  MSQ_ERR_SCRATCH = -3,     /* caller scratch smaller than *_scratch_bytes() */
  MSQ_ERR_HIP = -4          /* HIP runtime / launch error (text in msq_last_error) */
};

/* reference: ms::Buffer (src/core/metal.hpp:11-18): device allocation base, byte offset, usable bytes from off */
typedef struct MsqBuffer { void* dev; size_t off; size_t size; } MsqBuffer;

/* reference: ms::q::MvCfg (quant.hpp:12). Launch shape of the decode matvec, 0 = auto:
 * nr = rows one wave computes per tile, rsg = row-waves per workgroup, ks = waves splitting K inside a workgroup.
 * nr and rsg never change a row's summation order; ks does.
 * The environment can impose the same three values on every call, on top of a passed shape (reference:
 * MACSEEK_MV_NR / _RSG / _KS and MACSEEK_MVN_*, quant.mm:78-83,141): MSQ_MV_NR, MSQ_MV_RSG, MSQ_MV_KS for one token,
 * MSQ_MVN_NR, MSQ_MVN_RSG, MSQ_MVN_KS for msq_matvec_n with several; read once per process. */
typedef struct MsqMvCfg { int nr, rsg, ks; } MsqMvCfg;

/* Library / device bring-up (no reference counterpart: Metal pipelines are created lazily by ms::Device). Optional:
 * every entry point initialises on first use. Returns MSQ_OK or MSQ_ERR_HIP. */
int msq_init(void);
/* Last error message of the calling thread ("" if none). */
const char* msq_last_error(void);
/* 1 when the library was built for, and runs on, a gfx950 device. */
int msq_device_ok(void);

/* reference: block_elems / block_bytes / row_bytes / type_name (src/kernels/quant_types.hpp:13-43) */
int msq_block_elems(int qtype);
size_t msq_block_bytes(int qtype);
size_t msq_row_bytes(int qtype, int64_t cols);
const char* msq_type_name(int qtype);

/* reference: ms::q::matvec_supported (quant.hpp:14, quant.mm:68). Additionally true for IQ4_NL, for which the
 * reference has no GPU matvec (quant.mm:22-29). */
int msq_matvec_supported(int qtype);

/* reference: ms::q::matvec_cfg (quant.hpp:16-18, quant.mm:97-105): the launch shape msq_matvec would use. Row
 * chunks of one matrix that all pass this shape produce bit-identical rows. */
int msq_matvec_cfg(int qtype, int rows, int cols, MsqMvCfg* out);

/* reference: ms::q::encode_matvec (quant.hpp:29-30, quant.mm:70-95).
 * y[rows] (+)= W[rows x cols] . x[cols]; groups > 1 = block-diagonal: rows split into `groups` equal row groups,
 * group g reads x[g*cols .. g*cols + cols). cfg may be NULL. Errors (reference aborts): unsupported type,
 * cols not a multiple of the block size (256 for K/IQ/dense types, 32 for Q8_0 / IQ4_NL), groups < 1,
 * rows % groups != 0. */
int msq_matvec(void* stream, int qtype, const MsqBuffer* W, int rows, int cols, const MsqBuffer* x,
               const MsqBuffer* y, int accumulate, int groups, const MsqMvCfg* cfg);

/* reference: ms::q::encode_matvec_rmsnorm (quant.hpp:20-26, quant.mm:107-127; kernel q_mv_rn, quant_mv.metal:58-141).
 * y = W . (x * rsqrt(mean(x^2) + eps) * norm_w): the decode matvec with the input RMSNorm fused into the activation
 * loads. Bit-identical to msq_rmsnorm(x, norm_w, tmp, 1, cols, eps) followed by msq_matvec(tmp) with no imposed launch
 * shape, for every cols (the reference: for cols > 1024): each workgroup replays msq_rmsnorm's reduction exactly.
 * Types F32 F16 BF16 Q8_0 Q5_K Q6_K (as the reference) and IQ4_NL; no block-diagonal groups, no accumulate; rows of
 * up to about 15000 columns (the normalized row is staged in LDS). tiles_per_tg is accepted and ignored (workgroups
 * are persistent: every one computes the scale once). */
int msq_matvec_rmsnorm(void* stream, int qtype, const MsqBuffer* W, int rows, int cols, const MsqBuffer* x,
                       const MsqBuffer* norm_w, float eps, const MsqBuffer* y, int tiles_per_tg);

/* reference: ms::arch::encode_rmsnorm (src/kernels/arch.hpp:127-130; kernel arch_rmsnorm, src/kernels/arch_sample.metal:
 * 216-233). y[r] = x[r] * rsqrt(mean(x[r]^2) + eps) * w for `rows` rows of `dim` floats; w may be NULL (no weight);
 * strides in floats (0 = dim); y may alias x. */
int msq_rmsnorm(void* stream, const MsqBuffer* x, const MsqBuffer* w, const MsqBuffer* y, int rows, int dim, float eps,
                int in_stride, int out_stride);

/* reference: ms::q::encode_matvec_n (quant.hpp:32-35, quant.mm:129-156).
 * Y[n x rows] (+)= X[n x cols] . W^T for n in 1..16 (one weight read serves all n tokens). X row stride is
 * cols * groups, Y row stride is rows. n == 1 is exactly msq_matvec. For n >= 2, rows of up to 16384 columns (dense
 * types: 8192) run in a dot-product kernel that stages activations as fp16 pairs for the K / IQ formats (the
 * reference's numerics from two tokens on), fp32 for Q8_0 and the dense types, and decodes each weight once for up to
 * eight tokens. From nine tokens on (groups == 1, X 16-byte aligned) Q5_K, Q6_K, IQ1_S and IQ2_XXS, and Q6_K matrices
 * of 5 to 12 MB at eight tokens, run in msq_matmul's fused matrix-core kernel (activations rounded to fp16, exact
 * payloads, scales in fp32); like msq_matmul these calls sum K slices through a buffer inside the library and must be
 * enqueued on one stream at a time (MSQ_MVN_MM=0 keeps them in the dot-product kernel). The reference hands n >= 8 to
 * its matmul kernel the same way (quant.mm:133-137). Wider rows, and
 * more than eight tokens over a large IQ4_NL / Q8_0 / F16 / BF16 matrix, run on the matrix cores with activations
 * rounded to fp16 (BF16 weights: split into two bf16 terms) and exact weights. Wide F32 matrices, and wide
 * block-diagonal calls whose group size is not a multiple of 16 rows, are served as n decode matvecs. */
int msq_matvec_n(void* stream, int qtype, const MsqBuffer* W, int rows, int cols, const MsqBuffer* X,
                 const MsqBuffer* Y, int n, int accumulate, int groups);

/* reference: ms::q::encode_f32_to_f16 (quant.hpp:42, quant.mm:186-191). count % 4 == 0; X 16-byte aligned. */
int msq_f32_to_f16(void* stream, const MsqBuffer* X, const MsqBuffer* X16, size_t count);

/* reference: ms::q::encode_matmul_h (quant.hpp:43-45, quant.mm:193-238). Prefill matmul
 * Y[n x rows] (+)= X16[n x x_stride] . W^T, X16 fp16 (x_stride = cols if 0), Y F32, any n >= 1, cols % 128 == 0.
 * Weights are rounded to fp16 and products accumulate in fp32, the reference's numerics (quant.hpp:36-39).
 * Up to 128 tokens (256 on matrices of at most 2048 rows and on Q6_K / Q5_K; MSQ_MM_FUSED_MAX=N in the environment: up
 * to N) a fused kernel serves the call: nothing is allocated and the call only enqueues. When the matrix has few tiles K
 * is cut into slices whose partial sums pass through a 32 MB buffer inside the library and are added in order (results
 * repeat bit for bit; calls on this route share the buffer: one stream at a time). IQ1_S, IQ2_XXS, IQ4_NL and Q8_0
 * matrices of 12 million weights and more take a second fused kernel from 65 to 256 tokens, which stages both operands
 * through LDS (same numerics, same buffers; it wants activation rows on 16-byte boundaries, other strides stay with the
 * first kernel). Above, an fp16 copy of W goes to scratch that the library owns (reference: quant.mm:176-184): that
 * scratch only grows (a larger shape allocates a new block, never waits for the stream; inside a stream capture a call
 * that would have to grow it fails with MSQ_ERR_SCRATCH), and calls sharing it must be enqueued on one stream at a time. */
int msq_matmul_h(void* stream, int qtype, const MsqBuffer* W, int rows, int cols, const MsqBuffer* X16, const MsqBuffer* Y,
                 int n, int accumulate, int x_stride);

/* reference: ms::q::encode_matmul (quant.hpp:40-41, quant.mm:240-248): converts X (F32 [n x cols], 16-byte aligned)
 * into library-owned fp16 scratch, then msq_matmul_h; the first fused kernel reads the F32 activations as they are, the
 * second one an fp16 copy in a 16 MB buffer inside the library (shared like the partial sums; larger copies go to the
 * growing scratch). */
int msq_matmul(void* stream, int qtype, const MsqBuffer* W, int rows, int cols, const MsqBuffer* X, const MsqBuffer* Y, int n,
               int accumulate);

/* Whole-buffer dequantization to fp32, bit-exact with the reference's CPU dequantizer
 * (reference: ref::dequant_row, tests/ref/dequant.cpp:34-120; GPU relative: q_deq_f16, quant_mm.metal:143-154).
 * n_elems must be a multiple of the block size; out holds n_elems floats. */
int msq_dequant(void* stream, int qtype, const MsqBuffer* W, int64_t n_elems, const MsqBuffer* out);

/* Achievable-bandwidth probe: streams `bytes` (multiple of 16, base 16-byte aligned) from `src` with 128-bit loads and
 * writes one checksum word per workgroup to `sink` (>= 4096 bytes). The benchmark uses it as the measured-bandwidth
 * denominator next to the 8 TB/s nominal peak (reference: q_bw_read_f4 / q_bw_read_chunk, src/kernels/quant_bench.metal:5-31,
 * used by bench/qmatvec.mm:18-31). */
int msq_bw_probe(void* stream, const MsqBuffer* src, size_t bytes, const MsqBuffer* sink);

/* ---------------------------------------------------------------------------------------------- MoE, one token */

/* reference: kMaxRouted / kExpertDim / kExpertInter (quant.hpp:49). The reference hard-codes the expert shape; here
 * dim / inter travel in the argument structs and 0 selects the reference constants. */
#define MSQ_MAX_ROUTED 6
#define MSQ_EXPERT_DIM 5120
#define MSQ_EXPERT_INTER 2304

/* reference: ms::q::ExpertSlot (quant.hpp:51-53): gate [dim -> inter], up [dim -> inter], down [inter -> dim] */
typedef struct MsqExpertSlot { MsqBuffer gate, up, down; } MsqExpertSlot;

/* reference: ms::q::MoeDecodeArgs (quant.hpp:55-71), field for field, plus dim / inter.
 * Routed types: IQ1_S or IQ2_XXS (gate/up and down may differ). Shared type: Q6_K or Q8_0 as in the reference
 * (quant.mm:255-261), and additionally IQ2_XXS or IQ1_S. */
typedef struct MsqMoeDecodeArgs {
  int t_gate_up;   /* routed gate/up type */
  int t_down;      /* routed down type */
  int n_routed;    /* 0..MSQ_MAX_ROUTED */
  MsqExpertSlot slot[MSQ_MAX_ROUTED];
  MsqBuffer weights; /* F32[n_routed] routing weights, device memory, may be written by an earlier kernel */
  int has_shared;
  int t_shared;    /* shared expert type, weight 1 */
  MsqExpertSlot shared;
  MsqBuffer x;     /* F32[dim] */
  MsqBuffer y;     /* F32[dim], the result is ACCUMULATED into y */
  MsqBuffer scratch; /* >= msq_moe_decode_scratch_bytes(inter): F32 h[(MSQ_MAX_ROUTED + 1)][inter], then the same values
                      * as F16 (x 128, the form the down kernel multiplies; written for IQ1_S / IQ2_XXS down + shared) */
  /* launch shape overrides, 0 = default: rows per wave (nr) and row-waves per workgroup (rsg) of the gate/up and
   * down kernels. They never change a row's summation order (reference: quant.hpp:67-69). */
  int gu_nr, gu_rsg, d_nr, d_rsg;
  int dim, inter;  /* 0 = MSQ_EXPERT_DIM / MSQ_EXPERT_INTER; both multiples of 256, at most 32768 */
} MsqMoeDecodeArgs;

/* reference: ms::q::MoePart (quant.hpp:85): pieces of the table variant.
 *   SHARED_GU then AFTER_SHARED_GU == ALL, bit-identical
 *   SHARED then ROUTED             == ALL up to float summation order
 *   SHARED_GU then SHARED_DOWN     == SHARED, bit-identical */
enum { MSQ_PART_ALL = 0, MSQ_PART_SHARED_GU = 1, MSQ_PART_AFTER_SHARED_GU = 2, MSQ_PART_SHARED = 3,
       MSQ_PART_ROUTED = 4, MSQ_PART_SHARED_DOWN = 5,
       /* no reference counterpart: the two kernels of ALL on their own (GU then DOWN == ALL, bit-identical), so a
        * caller can time them separately or put other work between them */
       MSQ_PART_GU = 6, MSQ_PART_DOWN = 7 };

/* reference: ms::q::moe_decode_scratch_bytes (quant.hpp:72, quant.mm:264); inter = 0 means MSQ_EXPERT_INTER */
size_t msq_moe_decode_scratch_bytes(int inter);

/* reference: ms::q::encode_moe_decode (quant.hpp:73-75, quant.mm:266-315). Two kernels on the stream: gate + up +
 * SwiGLU (u = clamp(up, -10, 10), g = min(gate, 10), h = silu(g) * u * weight) for all experts, then down for all
 * experts accumulated into y. n_routed == 0 without a shared expert returns MSQ_OK and does nothing. */
int msq_moe_decode(void* stream, const MsqMoeDecodeArgs* a);

/* reference: ms::q::encode_moe_decode_table (quant.hpp:76-78, quant.mm:317-319). Routed matrices come from `table`:
 * MSQ_MAX_ROUTED entries of three device addresses {gate, up, down} (uint64), read by the GPU when the kernels run,
 * so the host may fill it after this call returned as long as it is complete before the GPU reaches the kernels.
 * a->slot[] is ignored. The table must be readable from the device (device or pinned host memory). */
int msq_moe_decode_table(void* stream, const MsqMoeDecodeArgs* a, const MsqBuffer* table);

/* reference: ms::q::encode_moe_decode_table_part (quant.hpp:79-86, quant.mm:321-369). SHARED_GU / SHARED /
 * SHARED_DOWN never read `table` (it may be NULL for them). */
int msq_moe_decode_table_part(void* stream, const MsqMoeDecodeArgs* a, const MsqBuffer* table, int part);

/* No counterpart in the reference. msq_moe_decode for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc): `a->scratch` is ignored, the h rows live in a
 * device array inside the library (7 x 4096 x 6 bytes = 168 KiB per GPU, held until the process ends), and the call
 * allocates nothing. inter above msq_moe_decode_static_max_inter() (4096) is refused with MSQ_ERR_SCRATCH. Every call
 * on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams) race; calls on one stream do not.
 * Results are bit-identical to msq_moe_decode with caller scratch. */
int msq_moe_decode_static(void* stream, const MsqMoeDecodeArgs* a);
int msq_moe_decode_static_max_inter(void);

/* ---------------------------------------------------------------------------------------------- MoE, prefill */

/* reference: ms::q::MoePrefillArgs (quant.hpp:93-116), field for field, plus dim / inter / x_is_bf16.
 * Routing is expert-sorted: routed expert j (0..n_exp-1, any subset of the layer's experts) owns entries
 * [offs[j], offs[j+1]) of tok[] (token row in X) and wt[] (routing weight). slot_of[t * k_per_token + k] is the entry
 * index of token t's k-th routed expert (-1 = none). Routed types: IQ1_S or IQ2_XXS; shared type: Q6_K, Q8_0, IQ2_XXS
 * or IQ1_S. */
typedef struct MsqMoePrefillArgs {
  int t_gate_up, t_down;
  int n_tokens;                 /* rows of X / Y */
  int n_exp;                    /* routed experts with >= 1 token */
  const MsqExpertSlot* slots;   /* host [n_exp] */
  const int* offs;              /* host [n_exp + 1], offs[0] = 0, offs[n_exp] = total entries */
  MsqBuffer tok;                /* device int32[total] */
  MsqBuffer wt;                 /* device F32[total] */
  MsqBuffer slot_of;            /* device int32[n_tokens * k_per_token] */
  int k_per_token;
  int has_shared;
  int t_shared;
  MsqExpertSlot shared;
  MsqBuffer X;                  /* F32 (or BF16 when x_is_bf16) [n_tokens x dim] */
  MsqBuffer Y;                  /* F32 [n_tokens x dim], ACCUMULATED */
  MsqBuffer scratch;            /* >= msq_moe_prefill_scratch_bytes(total, n_tokens, n_exp, dim, inter) */
  int path;                     /* reference kernel-family selector (quant.hpp:111-114): accepted, one family here */
  int shared_dense;             /* reference shared-expert route selector (quant.hpp:115): accepted, one route here */
  int dim, inter;               /* 0 = MSQ_EXPERT_DIM / MSQ_EXPERT_INTER; multiples of 256, at most 8192 */
  int x_is_bf16;                /* activations are bf16 instead of the reference's F32 */
} MsqMoePrefillArgs;

/* reference: ms::q::moe_prefill_scratch_bytes (quant.hpp:117, quant.mm:427-431). Layout (caller-owned device memory):
 * header (expert pointer table, offsets, token-tile table) | Xg fp16[(total+n) x dim] | H fp16[(total+n) x inter] |
 * Z f32[(total+n) x dim]. The header is written by small kernels that carry it in their arguments, so unlike the
 * reference the scratch may still be in use by earlier work on the same stream. */
size_t msq_moe_prefill_scratch_bytes(int total_entries, int n_tokens, int n_exp, int dim, int inter);

/* reference: ms::q::encode_moe_prefill (quant.hpp:118, quant.mm:433-612). Enqueues gather, grouped gate/up GEMM +
 * SwiGLU, grouped down GEMM and the ordered reduction into Y. Activations and H are staged as fp16 and weights enter
 * the matrix instructions as fp16 like the reference's tiles (IQ1_S / IQ2_XXS: the sub-block scale is rounded to fp16 and
 * its product with the grid value is rounded again, where the reference rounds the fp32 product once). The call only enqueues
 * (no host copy, no wait, no allocation) and can be captured in a HIP graph. Two of its launches are independent and
 * run side by side: one is forked onto a stream that the library owns (one per device, created by msq_init() or by the
 * first call outside a capture) and joined back before the call's later launches, all through events, so the caller
 * sees the ordering of a single stream (MSQ_MOEP_ONE_STREAM=1 in the environment turns the fork off); `offs` (host memory) is read at call time and
 * travels to the device inside kernel arguments. The result is bit-identical from run to run. n_tokens <= 0 returns MSQ_OK and
 * does nothing (quant.mm:435). */
int msq_moe_prefill(void* stream, const MsqMoePrefillArgs* a);

/* ---- router and routing lists: what produces the ids / weights of msq_moe_decode and the expert-sorted
 * tok / wt / slot_of / offs of msq_moe_prefill (reference module: src/kernels/arch.hpp:79-97) ---- */

/* reference: ms::arch::encode_router_topk (arch.hpp:84-85; kernel arch_router_topk, src/kernels/arch_router.metal:26-83;
 * CPU twin ref_arch::router, tests/ref/arch_ref.cpp:97-113). logits F32 [n_tokens][n_exp], bias F32 [n_exp] ->
 * ids int32 [n_tokens][6], w F32 [n_tokens][6], descending by key = sqrt(softplus(logit)) + bias, ties to the lower
 * expert id; w = score / (sum of the six scores + 1e-20) * route_scale (the reference fixes n_exp = 384 and
 * route_scale = 1.5; here n_exp is a multiple of 64 up to 512). n_tokens == 0 does nothing. */
int msq_router_topk(void* stream, const MsqBuffer* logits, const MsqBuffer* bias, const MsqBuffer* ids, const MsqBuffer* w,
                    int n_tokens, int n_exp, float route_scale);

/* reference: ms::arch::encode_router_fused (arch.hpp:79-83; kernel arch_router_fused, arch_router.metal:86-121):
 * logits = W[n_exp][dim] . x[dim] and the selection in one launch; W is F32 (the reference's ffn_gate_inp) or BF16.
 * scratch (>= msq_router_scratch_bytes(n_exp), the reference's Scratch::router_logits + counter) receives the logits in
 * its first n_exp floats; the caller zeroes it once before the first call and the call leaves its counter re-armed.
 * A scratch belongs to one stream at a time: calls sharing it must not overlap. A launch that fails (MSQ_ERR_HIP) or is
 * torn down part-way may leave the counter between zero and the workgroup count, after which calls would select
 * nothing: zero the scratch again before it is reused. */
size_t msq_router_scratch_bytes(int n_exp);
int msq_router_fused(void* stream, int wtype, const MsqBuffer* x, const MsqBuffer* W, const MsqBuffer* bias,
                     const MsqBuffer* scratch, const MsqBuffer* ids, const MsqBuffer* w, int dim, int n_exp,
                     float route_scale);

/* reference: ms::arch::RouteLists (arch.hpp:87-96): device buffers for up to max_tokens tokens. */
typedef struct {
  MsqBuffer counts;  /* u32 [n_exp] */
  MsqBuffer offsets; /* u32 [n_exp + 1] exclusive scan, offsets[n_exp] = number of entries with a valid id */
  MsqBuffer entry;   /* u32 [6 n] entry index t * 6 + k */
  MsqBuffer tok;     /* u32 [6 n] token t */
  MsqBuffer w;       /* f32 [6 n] routing weight */
  MsqBuffer slot_of; /* u32 [6 n] position of entry t * 6 + k in the sorted lists */
  int max_tokens;
} MsqRouteLists;

/* reference: ms::arch::encode_route_lists (arch.hpp:97; kernels arch_route_count / arch_route_scatter,
 * arch_router.metal:124-183; CPU twin ref_arch::route_lists, tests/ref/arch_ref.cpp:114-130). Entries (t, k) = t * 6 + k
 * sorted by expert, then entry index; no atomics, so the lists are identical on every run. tok / w / slot_of / offsets
 * are the tok / wt / slot_of / offs inputs of msq_moe_prefill. Entries whose id is outside 0..n_exp-1 are left out
 * (their slot_of is not written). */
int msq_route_lists(void* stream, const MsqBuffer* ids, const MsqBuffer* w, int n_tokens, int n_exp, const MsqRouteLists* L);

/* ---- GGUF reader and resident expert placement: the on-disk format on the input side of the kernels ---- */

/* reference: ms::Gguf (src/gguf/gguf.hpp:38-96, src/gguf/gguf.cpp). Opaque handle over one model: one file, or all M
 * splits when the path matches "*-0000N-of-0000M.gguf". GGUF versions 2 and 3. Metadata is merged across splits (the
 * first occurrence wins); tensors are listed in file order, split by split, with ABSOLUTE file offsets. Pure host
 * code: nothing here touches the GPU except msq_gguf_load_tensor and msq_gguf_place_experts. */
typedef struct MsqGguf MsqGguf;
int msq_gguf_open(const char* path, MsqGguf** out);
void msq_gguf_close(MsqGguf* g);
int msq_gguf_n_splits(const MsqGguf* g);
int msq_gguf_n_tensors(const MsqGguf* g);
int msq_gguf_n_kv(const MsqGguf* g);
uint32_t msq_gguf_alignment(const MsqGguf* g); /* general.alignment of the first split, 32 if absent */
uint32_t msq_gguf_version(const MsqGguf* g);
const char* msq_gguf_split_path(const MsqGguf* g, int split);
uint64_t msq_gguf_data_offset(const MsqGguf* g, int split);
int msq_gguf_split_count_of_path(const char* path); /* reference: Gguf::expand_splits(path).size() */

/* reference: ms::type_bytes / ms::type_name (gguf.hpp:19-22): every ggml type id, also those the kernels do not take */
uint64_t msq_gguf_type_bytes(int ggml_type, uint64_t n_elems);
const char* msq_gguf_type_name(int ggml_type); /* "?" if unknown */

/* reference: ms::TensorInfo (gguf.hpp:40-51); name stays valid until msq_gguf_close */
typedef struct {
  const char* name;
  int type;      /* ggml type id */
  int n_dims;
  int64_t ne[4]; /* ggml order: ne[0] contiguous (= cols of a weight matrix), ne[1] = rows, ne[2] = experts */
  uint64_t nbytes;
  int split;
  uint64_t offset; /* absolute byte offset of the data in that split file */
} MsqGgufTensor;
int msq_gguf_tensor(const MsqGguf* g, int index, MsqGgufTensor* out);
int msq_gguf_find(const MsqGguf* g, const char* name); /* index, or -1 */

/* metadata; value types as in the container: 0 u8, 1 i8, 2 u16, 3 i16, 4 u32, 5 i32, 6 f32, 7 bool, 8 string, 9 array,
 * 10 u64, 11 i64, 12 f64. Getters return the default for a missing key or a mismatched kind (gguf.hpp:66-71). */
const char* msq_gguf_key(const MsqGguf* g, int index); /* insertion order */
int msq_gguf_kv_type(const MsqGguf* g, const char* key, int* arr_type); /* -1 if missing; *arr_type = element type or -1 */
int64_t msq_gguf_get_i64(const MsqGguf* g, const char* key, int64_t dflt);
double msq_gguf_get_f64(const MsqGguf* g, const char* key, double dflt);
const char* msq_gguf_get_str(const MsqGguf* g, const char* key, const char* dflt);
int64_t msq_gguf_arr_len(const MsqGguf* g, const char* key); /* -1 if missing or not an array */
int64_t msq_gguf_arr_i64(const MsqGguf* g, const char* key, int64_t* out, int64_t cap); /* values written */
int64_t msq_gguf_arr_f64(const MsqGguf* g, const char* key, double* out, int64_t cap);
const char* msq_gguf_arr_str(const MsqGguf* g, const char* key, int64_t index);
int64_t msq_gguf_arr_nested_i64(const MsqGguf* g, const char* key, int64_t index, int64_t* out, int64_t cap); /* inner length */

/* reference: ms::pread_full on the tensor's split (gguf.hpp:99): bytes [byte_off, byte_off + len) of the tensor's data
 * into host memory; returns the bytes read, -1 on a bad range. */
int64_t msq_gguf_read(const MsqGguf* g, int tensor, uint64_t byte_off, void* dst, uint64_t len);
/* The same range into device memory (pinned staging, copies enqueued on `stream`; returns after the last chunk has been
 * read from the file and copied). */
int msq_gguf_load_tensor(void* stream, const MsqGguf* g, int tensor, uint64_t byte_off, uint64_t len, const MsqBuffer* dst);

/* reference: ms::ExpertLayout::from_gguf for one layer (src/store/experts.hpp:35-42, src/store/experts.mm:36-56):
 * index k = 0 gate (blk.L.ffn_gate_exps.weight), 1 up, 2 down; stride = nbytes / n_experts, the per-expert slab. */
typedef struct {
  int n_experts;
  int type[3];         /* ggml type of the gate / up / down matrices */
  int64_t rows[3], cols[3];
  uint64_t stride[3];  /* bytes of one expert's matrix */
  int tensor[3];       /* tensor indices */
  uint64_t arena_bytes; /* device bytes msq_gguf_place_experts needs: every slab padded to 256 bytes */
} MsqExpertLayout;
int msq_gguf_expert_layout(const MsqGguf* g, int layer, MsqExpertLayout* out);

/* Resident placement of one layer's experts (no reference counterpart: the reference streams experts from SSD into a
 * cache arena, src/store/experts.hpp:60-250; an MI355X keeps them all in HBM). Copies the three stacked tensors into
 * `arena` (device memory, 256-byte aligned, >= arena_bytes), every expert matrix at a 256-byte aligned offset, and
 * fills slots[e] (e < n_experts <= n_slots) with views of it for msq_moe_decode / msq_moe_prefill. */
int msq_gguf_place_experts(void* stream, const MsqGguf* g, int layer, const MsqBuffer* arena, MsqExpertSlot* slots, int n_slots);

#ifdef __cplusplus
}
#endif
#endif /* MSQ_H */
