/*
 * gmlp.h — C ABI of libgmlp.so: gated-MLP forward/backward kernels for AMD Instinct MI355X (gfx950).
 *
 * The library is the device half of a drop-in for the operator layer of matteobonotto/triton-gated-mlp.
 * Every entry point below names the reference interface it stands behind (paths relative to the
 * reference repository root).  The reference launches Triton JIT kernels from Python; here the same
 * host wrappers load this library with ctypes and pass raw device pointers.
 *
 * Conventions
 *   - All matrices are dense, row-major, contiguous, on the current HIP device, 16-byte aligned.
 *   - M = tokens (rows of x), K = hidden_size, N = intermediate_size.
 *     W_gate, W_up are [N,K]; W_down is [K,N]  (torch.nn.Linear [out,in] layout).
 *   - dtype: GMLP_F16 or GMLP_BF16 storage (the tuned kernels) or GMLP_F32 (compatibility path on
 *     fp32 MFMA, not tuned; not for gmlp_decode_fwd); accumulation and epilogue arithmetic are fp32.
 *   - Every call only ENQUEUES work on `stream` (a hipStream_t; NULL = default stream) and returns.
 *     The library never allocates or frees device memory and keeps no pointer past a call; the
 *     caller owns every buffer, including workspaces (sizes from gmlp_workspace_bytes).  The one
 *     piece of device memory of its own is the static scratch array of gmlp_colsum_static.
 *   - Return value: 0 on success, a negative GMLP_E* code otherwise; nothing is launched on error.
 *     gmlp_last_error() returns a thread-local message for the last failing call on this thread.
 *   - Dropout: keep(m,n) = philox4x32_10(counter = {lo32(e/4), hi32(e/4), lo32(offset), hi32(offset)},
 *     key = {lo32(seed), hi32(seed)})[e%4] >= floor(p * 2^32), with e = m*N + n; kept values are
 *     scaled by 1/(1-p).  p == 0 disables dropout (the generator is not evaluated).
 */
#ifndef GMLP_H_
#define GMLP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GMLP_ABI_VERSION 8

enum gmlp_dtype { GMLP_F16 = 0, GMLP_BF16 = 1, GMLP_F32 = 2 };

/*
 * Gate activation `act` of the hidden state H = act(G) ⊙ U.  The functions are those of the
 * reference's hidden_act table (ACT2CLS / ACT_FWD, src/triton_gated_mlp/gated_mlp.py:17-37) with
 * torch's default parameters: exact (erf) GELU, LeakyReLU slope 0.01; "swish" is GMLP_ACT_SILU and
 * "no_act" is GMLP_ACT_IDENTITY.  The reference's fused kernels implement silu and no_act only
 * (_act_fwd/_act_bwd, src/triton_gated_mlp/ops/act.py:5-22); derivatives here are the true ones
 * (identity' = 1, relu'(0) = 0, leaky_relu'(0) = 0.01, as torch.autograd).
 */
enum gmlp_act {
  GMLP_ACT_SILU = 0,
  GMLP_ACT_GELU = 1,
  GMLP_ACT_RELU = 2,
  GMLP_ACT_LEAKY_RELU = 3,
  GMLP_ACT_SIGMOID = 4,
  GMLP_ACT_TANH = 5,
  GMLP_ACT_IDENTITY = 6
};

enum gmlp_status {
  GMLP_OK = 0,
  GMLP_EINVAL = -1, /* null pointer, bad dtype or act code, bad dropout probability */
  GMLP_ESHAPE = -2, /* shape not supported (see each entry point) */
  GMLP_EALIGN = -3, /* pointer not 16-byte aligned */
  GMLP_EHIP = -4    /* HIP runtime reported an error at launch */
};

enum gmlp_op {
  GMLP_OP_DECODE_FWD = 0,
  GMLP_OP_COLSUM = 1,
  GMLP_OP_LINEAR_FWD = 2,
  GMLP_OP_DX_BWD = 3,
  GMLP_OP_GATEUP_FWD = 4,
  GMLP_OP_DH_BWD = 5,
  GMLP_OP_DW_BWD = 6,
  GMLP_OP_DW_BWD_GROUPED = 7
};

int gmlp_abi_version(void);
const char* gmlp_last_error(void);

/*
 * Optional set-up for the current HIP device: makes every one-time runtime call the entry points
 * would otherwise make at their first launch on that device (raising the dynamic-LDS limit of each
 * kernel, reading the compute-unit count, resolving the address of the static scratch array of
 * gmlp_colsum_static).  Call it once per device before capturing a stream into a HIP graph: those
 * calls are not allowed during capture, and an entry point that still needs one while its stream
 * is capturing returns GMLP_EHIP (hipErrorStreamCaptureUnsupported) instead of making it.
 * No counterpart in the reference (Triton compiles and configures its kernels at first launch,
 * src/triton_gated_mlp/ops/fwd.py:257-276).
 */
int gmlp_init(void);

/*
 * Workspace bytes the caller must provide for `op` at the given problem size (0 if none), with
 * (M, K, N) as the entry point of that name takes them: GMLP_OP_COLSUM (M, 0, C),
 * GMLP_OP_LINEAR_FWD (M, R, C), GMLP_OP_DX_BWD (M, K, N), GMLP_OP_GATEUP_FWD (M, K, N),
 * GMLP_OP_DECODE_FWD (M, K, N), GMLP_OP_DH_BWD (M, K, N), GMLP_OP_DW_BWD (Mred, R, C),
 * GMLP_OP_DW_BWD_GROUPED (arguments ignored: an upper bound for any set of problems, 128 MiB on a
 * whole MI355X).  The values are enumerators, not flags: ask per operation; one buffer of the
 * largest answer serves every call of a forward or backward pass (calls on one stream are ordered).
 * Two things use a workspace, and without one (NULL, 0) every entry point computes the same result
 * more slowly on the shapes concerned: split reductions for short batches (see gmlp_linear_fwd),
 * and stream-K for grids of large tiles that end in a thinly filled round of workgroups while the
 * reduction is long (the last round's tiles are then shared out by reduction range over all compute
 * units, fp32 partial sums pass through the workspace and a second launch adds them up in a fixed
 * order: results do not depend on timing).
 */
size_t gmlp_workspace_bytes(int op, int64_t M, int64_t K, int64_t N, int dtype);

/*
 * Hidden-state forward:  G = x·W_gateᵀ + b_gate,  U = x·W_upᵀ + b_up,
 *                        H = dropout(act(G) ⊙ U).
 * Replaces mlp_hidden_states_fwd + _fwd_kernel (src/triton_gated_mlp/ops/fwd.py:198-279, :72-166);
 * math of EagerGatedMLP.forward (src/triton_gated_mlp/gated_mlp.py:96) and eager_fwd (:105-128).
 * b_gate, b_up, g_save, u_save, mask_out may be NULL.  g_save/u_save [M,N] receive G and U
 * (activations kept for the backward pass).  mask_out [M,N] uint8 receives the keep mask.
 * Requires K % 8 == 0, N % 8 == 0, M >= 1.
 * workspace (may be NULL): gmlp_workspace_bytes(GMLP_OP_GATEUP_FWD, M, K, N, dtype) bytes, used as
 * in gmlp_linear_fwd (non-zero for short batches whose tiles would leave half the chip idle).
 */
int gmlp_gateup_fwd(const void* x, const void* w_gate, const void* w_up, const void* b_gate,
                    const void* b_up, void* h, void* g_save, void* u_save, uint8_t* mask_out,
                    int64_t M, int64_t K, int64_t N, int dtype, int act, float dropout_p,
                    uint64_t seed, uint64_t offset, void* workspace, size_t workspace_bytes,
                    void* stream);

/*
 * Linear layer forward: out[M,C] = a[M,R]·w[C,R]ᵀ + bias[C]   (bias may be NULL).
 * Replaces the nn.Linear down_proj call (src/triton_gated_mlp/gated_mlp.py:236), which the
 * reference leaves to the vendor BLAS.  Requires R % 8 == 0, C % 8 == 0.
 * workspace (may be NULL): gmlp_workspace_bytes(GMLP_OP_LINEAR_FWD, M, R, C, dtype) bytes.  It is
 * non-zero for outputs of a few tiles with a long reduction (short batches): with it the reduction
 * is split over several workgroups per tile (fp32 partial sums, added in a fixed order); without
 * it the same result comes from one workgroup per tile, several times slower on such shapes.
 */
int gmlp_linear_fwd(const void* a, const void* w, const void* bias, void* out, int64_t M, int64_t R,
                    int64_t C, int dtype, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Backward through down_proj, dropout and the gating product in one GEMM:
 *   dH = dY·W_down ; dA = dH ⊙ keep/(1-p) ; dU = dA ⊙ act(G) ; dG = dA ⊙ U ⊙ act'(G).
 * Replaces the autograd backward of down_proj plus _compute_quantities_for_bwd
 * (src/triton_gated_mlp/ops/bwd.py:89-211; closed form in gated_mlp.py:131-144).  g, u are the
 * tensors written by gmlp_gateup_fwd (g_save, u_save).  dg, du are [M,N].
 * workspace (may be NULL): gmlp_workspace_bytes(GMLP_OP_DH_BWD, M, K, N, dtype) bytes.
 */
int gmlp_dh_bwd(const void* dy, const void* w_down, const void* g, const void* u, void* dg, void* du,
                int64_t M, int64_t K, int64_t N, int dtype, int act, float dropout_p, uint64_t seed,
                uint64_t offset, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Element-wise gating backward for callers that already hold dH (the reference's operator-level
 * backward receives grad_output = dH):  dU = dA ⊙ act(G), dG = dA ⊙ U ⊙ act'(G), dA as above.
 * Replaces the epilogue of _compute_quantities_for_bwd (src/triton_gated_mlp/ops/bwd.py:196-211).
 */
int gmlp_gating_bwd(const void* dh, const void* g, const void* u, void* dg, void* du, int64_t M,
                    int64_t N, int dtype, int act, float dropout_p, uint64_t seed, uint64_t offset,
                    void* stream);

/*
 * dX = dG·W_gate + dU·W_up   (one GEMM over the concatenated reduction of length 2N).
 * Replaces _compute_dx (src/triton_gated_mlp/ops/bwd.py:242-322; gated_mlp.py:147-149).
 * workspace (may be NULL): gmlp_workspace_bytes(GMLP_OP_DX_BWD, M, K, N, dtype) bytes, used as in
 * gmlp_linear_fwd.
 */
int gmlp_dx_bwd(const void* dg, const void* du, const void* w_gate, const void* w_up, void* dx,
                int64_t M, int64_t K, int64_t N, int dtype, void* workspace, size_t workspace_bytes,
                void* stream);

/*
 * Weight gradient: dw[R,C] = lhs[Mred,R]ᵀ · rhs[Mred,C].
 * Replaces _compute_dW_up_dW_gp (src/triton_gated_mlp/ops/bwd.py:386-463; gated_mlp.py:152-155)
 * with (lhs,rhs) = (dG,x), (dU,x); and the autograd dW of down_proj with (lhs,rhs) = (dY,H).
 * Requires R % 8 == 0, C % 8 == 0.
 * workspace (may be NULL): gmlp_workspace_bytes(GMLP_OP_DW_BWD, Mred, R, C, dtype) bytes.
 */
int gmlp_dw_bwd(const void* lhs, const void* rhs, void* dw, int64_t Mred, int64_t R, int64_t C,
                int dtype, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Up to 3 weight gradients that share the reduction length Mred, enqueued as ONE grid when every
 * problem fits the full-tile kernel (otherwise as `count` separate launches):
 *   dw[i][R[i],C[i]] = lhs[i][Mred,R[i]]ᵀ · rhs[i][Mred,C[i]],  i < count.
 * Same reference counterparts as gmlp_dw_bwd; one launch for dW_gate, dW_up and dW_down avoids
 * three partially filled last rounds of workgroups.
 * workspace (may be NULL): gmlp_dw_bwd_grouped_workspace_bytes(count, Mred, R, C, dtype) bytes (what
 * this set of problems uses, often 0), or the bound gmlp_workspace_bytes(GMLP_OP_DW_BWD_GROUPED, ...).
 */
size_t gmlp_dw_bwd_grouped_workspace_bytes(int count, int64_t Mred, const int64_t* R, const int64_t* C,
                                           int dtype);
int gmlp_dw_bwd_grouped(int count, const void* const* lhs, const void* const* rhs, void* const* dw,
                        int64_t Mred, const int64_t* R, const int64_t* C, int dtype, void* workspace,
                        size_t workspace_bytes, void* stream);

/*
 * Bias gradient: out[C] = Σ_m a[m,C], fp32 accumulation in a fixed order (deterministic).
 * workspace: gmlp_workspace_bytes(GMLP_OP_COLSUM, M, 0, C, dtype) bytes.
 * The reference returns None for bias gradients (gated_mlp.py:200); EagerGatedMLP's autograd
 * produces them, and this entry point supplies them.
 */
int gmlp_colsum(const void* a, void* out, void* workspace, int64_t M, int64_t C, int dtype,
                void* stream);

/*
 * gmlp_colsum for callers that cannot allocate device memory (code running under HIP graph capture,
 * serving loops and harnesses that forbid allocation): the same kernels and the same result, bit
 * for bit, with the first stage's partial sums kept in a static device array of the library instead
 * of a caller's workspace.  It has no counterpart in the reference.  The array holds
 * 64 x GMLP_COLSUM_STATIC_MAX_C floats (8 MiB) on every GPU the library has run on, until the
 * process ends; C beyond GMLP_COLSUM_STATIC_MAX_C is rejected with GMLP_ESHAPE.  The call makes no
 * hipMalloc/hipFree.  Every call on a GPU uses that GPU's one array: calls that may overlap on one
 * GPU (different streams, or graphs replayed concurrently) race and must be serialised by the
 * caller; calls on one stream are ordered.  Nothing has to be cleared between calls: the first
 * stage overwrites every partial sum the second stage reads.
 */
#define GMLP_COLSUM_STATIC_MAX_C 32768
int gmlp_colsum_static(const void* a, void* out, int64_t M, int64_t C, int dtype, void* stream);

/*
 * Up to 3 bias gradients of one backward pass in one pair of launches: out[i][C[i]] = Σ_m a[i][m,C[i]].
 * workspace: the sum over i of gmlp_workspace_bytes(GMLP_OP_COLSUM, M, 0, C[i], dtype) bytes.
 * Same reference counterpart as gmlp_colsum.
 */
int gmlp_colsum_grouped(int count, const void* const* a, void* const* out, void* workspace, int64_t M,
                        const int64_t* C, int dtype, void* stream);

/*
 * Skinny-M forward of the whole MLP (decode): y = (act(x·W_gateᵀ+b_g) ⊙ (x·W_upᵀ+b_u))·W_downᵀ + b_d
 * for M <= 32, streaming each weight matrix from HBM exactly once.  h_scratch holds 16*N elements
 * of dtype for M <= 16 and 32*N beyond: the intermediate H for 16 or 32 token slots, in an order of
 * the library's choosing;
 * workspace: unused by the current kernels (gmlp_workspace_bytes(GMLP_OP_DECODE_FWD, ...) is 0): pass
 * NULL.  The argument is kept so that the signature does not change.  No dropout (inference).
 * Same math as EagerGatedMLP.forward in eval mode (src/triton_gated_mlp/gated_mlp.py:92-98).
 * Requires K % 32 == 0 and N % 256 == 0 (the LDS-ring streaming kernels run when K % 256 == 0 too,
 * K >= 768, N >= 768 and K*N < 2^30; 16 < M <= 32 is accepted only then).
 */
int gmlp_decode_fwd(const void* x, const void* w_gate, const void* w_up, const void* w_down,
                    const void* b_gate, const void* b_up, const void* b_down, void* h_scratch,
                    void* y, void* workspace, int64_t M, int64_t K, int64_t N, int dtype, int act,
                    void* stream);

/*
 * A whole pass of the MLP in one call: validates once and enqueues every launch of the pass, so a
 * host that drives the MLP from an interpreter pays for one foreign call per pass instead of one
 * per GEMM (a step of a small MLP is otherwise bound by the time it takes to enqueue it).
 *
 * gmlp_mlp_fwd:  H = dropout(act(x·W_gateᵀ + b_gate) ⊙ (x·W_upᵀ + b_up)),  y = H·W_downᵀ + b_down
 *   = gmlp_gateup_fwd followed by gmlp_linear_fwd, bit for bit.  Stands behind FusedGatedMLP.forward
 *   (src/triton_gated_mlp/gated_mlp.py:230-237: FusedGatedMLPFunction.apply, then down_proj) and
 *   mlp_hidden_states_fwd (src/triton_gated_mlp/ops/fwd.py:198-279).  h [M,N] is always written
 *   (it is the down projection's operand); g_save, u_save [M,N] and the biases may be NULL.
 *
 * gmlp_mlp_bwd: every gradient of the MLP from dy [M,K]:
 *   dG, dU (gmlp_dh_bwd) -> dx (gmlp_dx_bwd), dw_gate, dw_up, dw_down (gmlp_dw_bwd_grouped),
 *   db_gate, db_up, db_down (gmlp_colsum_grouped), the same values as those calls give.
 *   Stands behind mlp_hidden_states_bwd (src/triton_gated_mlp/ops/bwd.py:466-602, one host function
 *   that enqueues the whole hidden-state backward) plus the autograd backward of down_proj.
 *   g, u, h are what the forward pass left in g_save, u_save, h.  dg, du [M,N] are scratch the
 *   caller provides (they hold dG and dU on return).  Any output pointer may be NULL: that gradient
 *   is not computed, and what only it needs is not read (with dx, dw_gate, dw_up, db_gate and
 *   db_up all NULL nothing behind dG, dU runs and w_down, g, u, dg, du may be NULL too).
 *   Every launch goes to `stream`, in that order.
 *
 * workspace: gmlp_mlp_workspace_bytes(GMLP_PASS_FWD or GMLP_PASS_BWD, M, K, N, dtype) bytes (may be
 * NULL or smaller for a pass without bias gradients: launches then take their plain form, with the
 * same results up to the order of fp32 additions; bias gradients need it and fail with GMLP_EINVAL
 * without).
 */
enum gmlp_pass { GMLP_PASS_FWD = 0, GMLP_PASS_BWD = 1 };
size_t gmlp_mlp_workspace_bytes(int pass, int64_t M, int64_t K, int64_t N, int dtype);
int gmlp_mlp_fwd(const void* x, const void* w_gate, const void* w_up, const void* w_down, const void* b_gate,
                 const void* b_up, const void* b_down, void* y, void* h, void* g_save, void* u_save, int64_t M,
                 int64_t K, int64_t N, int dtype, int act, float dropout_p, uint64_t seed, uint64_t offset,
                 void* workspace, size_t workspace_bytes, void* stream);
int gmlp_mlp_bwd(const void* dy, const void* x, const void* w_gate, const void* w_up, const void* w_down,
                 const void* g, const void* u, const void* h, void* dg, void* du, void* dx, void* dw_gate,
                 void* dw_up, void* dw_down, void* db_gate, void* db_up, void* db_down, int64_t M, int64_t K,
                 int64_t N, int dtype, int act, float dropout_p, uint64_t seed, uint64_t offset, void* workspace,
                 size_t workspace_bytes, void* stream);

/* Writes the dropout keep mask (1 = keep) for an [M,N] tensor; the test oracle of the generator. */
int gmlp_dropout_mask(uint8_t* mask, int64_t M, int64_t N, float dropout_p, uint64_t seed,
                      uint64_t offset, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* GMLP_H_ */
