/*
 * C ABI of libf3d_hip.so — the gfx950 (MI355X) implementation of the Flash3D forward hot path.
 *
 * Every entry point is what a host binding for this path binds: plain pointers to DEVICE memory
 * (unless a parameter says "host"), sizes, and the HIP stream to launch on (`stream` is a
 * hipStream_t passed as void*, nullptr = the default stream).  Outputs are caller-allocated and
 * written in place, exactly as the reference's pybind functions do with at::Tensor& arguments
 * (src/f3d_frontend.cu:38-105).  All calls are asynchronous on `stream` unless
 * f3d_set_sync_stream(1) is in force.
 *
 * Return value: F3D_OK, or an error code with a message available from f3d_last_error().  Argument
 * violations mirror the reference's `throw std::runtime_error` sites; the host binding turns a
 * non-zero return into its language's exception.
 *
 * Types on the wire (reference: CoordT=fp16, CounterT=uint32, HashT=uint16, FeatT=bf16,
 * src/psh/batch_psh_bucket_dispatcher.cu:252-254, src/psh/batch_subbuck_pooling_dispatcher.cu:45-48):
 *   f3d_half_t  IEEE binary16 bit pattern          f3d_bf16_t  bfloat16 bit pattern
 */
#ifndef F3D_HIP_H
#define F3D_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint16_t f3d_half_t;
typedef uint16_t f3d_bf16_t;

#define F3D_OK 0
#define F3D_ERR_INVALID 1     /* bad argument (reference: std::runtime_error from a dispatcher) */
#define F3D_ERR_UNSUPPORTED 2 /* no kernel for this configuration (reference: "No kernel found") */
#define F3D_ERR_RUNTIME 3     /* HIP runtime failure */

/* hash_type values, src/psh/hash_fns.cuh:151-158 */
#define F3D_H_ZORDER_DIV 1
#define F3D_H_XORSUM_DIV 2
#define F3D_H_ZORDER_MOD 3
#define F3D_H_XORSUM_MOD 4

/* reduction ops, src/psh/batch_psh_subbuck_reduce.cuh:47-52 */
#define F3D_O_MEAN 0
#define F3D_O_SUM 1
#define F3D_O_MIN 2
#define F3D_O_MAX 3

/* activation / epilogue selectors of f3d_linear_bf16 */
#define F3D_ACT_NONE 0
#define F3D_ACT_GELU 1   /* exact erf GELU */
#define F3D_ACT_SWIGLU 2 /* out[:, j] = silu(acc[:, j]) * acc[:, j + N/2]; output has N/2 columns */
#define F3D_ACT_SILU 3
#define F3D_ACT_RELU 4

/* ---- module state: DeviceManagerSingleton, src/common/device_manager.cu:58-119,
 *      src/f3d_frontend.cu:115-120 ------------------------------------------------------------ */

const char* f3d_last_error(void);      /* message of the last failing call on this thread */
int f3d_init_dev_info(int device);     /* init_dev_info: per-device one-time setup (idempotent) */
int f3d_set_sync_stream(int enable);   /* set_sync_stream: returns the new value */
int f3d_get_sync_stream(void);         /* get_sync_stream */
/* Seed of the stateless generator behind the sub-bucket rotation and the overflow probes.  The
 * reference seeds cuRAND with 3407 (device_manager.cu:66); same default here. */
int f3d_set_seed(uint32_t seed);
uint32_t f3d_get_seed(void);

/* ---- PSH bucketing: batch_psh_scatter_pad_hash, src/f3d_frontend.cu:52-58,
 *      src/psh/batch_psh_bucket_dispatcher.cu:221-326 ------------------------------------------
 * coord [total_n,3] fp16; bucket_id [total_n] u16; bucket_counter, cumsum_counter
 * [batch_size,num_bucket] u32 (bucket_counter is accumulated into: zero it first);
 * bucket_offset [total_n] u32; batch_sep [batch_size] u32 inclusive cumulative sizes;
 * bbox_min/max [3] fp16; probe_offsets [128,3] i16 (may be NULL when rebalancing is off);
 * scatter_coord [pad_to_n,3] fp16; rows [total_n,pad_to_n) receive pad_num.
 * Slots inside a bucket follow input order (the reference's order is arbitration-dependent).
 * Uses the per-device workspace: not re-entrant per device. */
int f3d_batch_psh_scatter_pad_hash(const f3d_half_t* coord, uint16_t* bucket_id, uint32_t* bucket_counter,
                                   uint32_t* bucket_offset, const uint32_t* batch_sep, uint32_t batch_size,
                                   uint32_t total_n, uint32_t instance_max_n, uint32_t num_bucket,
                                   uint32_t bucket_divisor, uint32_t bucket_size, uint32_t num_vox,
                                   const f3d_half_t* bbox_min, const f3d_half_t* bbox_max,
                                   const int16_t* probe_offsets, uint32_t* cumsum_counter,
                                   f3d_half_t* scatter_coord, uint32_t pad_to_n, float pad_num,
                                   uint32_t hash_type, int device, void* stream);

/* The same op for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  No counterpart in the reference.  Same arguments, same results bit for bit; the
 * tile histograms, first-hash counts and rebalance plan live in a fixed array of F3D_PSH_NOALLOC_SCRATCH_BYTES that
 * every GPU the library runs on holds until the process ends, instead of the library's grow-only workspace.  The
 * call makes no hipMalloc / hipFree and calls no allocating routine.  A batch that needs more scratch memory
 * (about batch_size * tiles_per_cloud * num_bucket 32-bit words; 4 clouds x 250,000 points need 4.1 MB, 64 clouds x
 * 262,144 points 4.7 MB) is rejected with F3D_ERR_UNSUPPORTED and a message.  The array's per-device
 * address is looked up once per device: by f3d_init_dev_info(device), else by the first call on that device (call
 * f3d_init_dev_info before a stream capture).  All calls on one GPU share the array, so calls that overlap on one
 * GPU (two streams, two threads) race; calls ordered on one stream do not.  Nothing in it needs clearing between
 * calls: every word a launch reads was written earlier in the same call. */
#define F3D_PSH_NOALLOC_SCRATCH_BYTES (8u << 20)
int f3d_batch_psh_scatter_pad_hash_noalloc(const f3d_half_t* coord, uint16_t* bucket_id, uint32_t* bucket_counter,
                                           uint32_t* bucket_offset, const uint32_t* batch_sep, uint32_t batch_size,
                                           uint32_t total_n, uint32_t instance_max_n, uint32_t num_bucket,
                                           uint32_t bucket_divisor, uint32_t bucket_size, uint32_t num_vox,
                                           const f3d_half_t* bbox_min, const f3d_half_t* bbox_max,
                                           const int16_t* probe_offsets, uint32_t* cumsum_counter,
                                           f3d_half_t* scatter_coord, uint32_t pad_to_n, float pad_num,
                                           uint32_t hash_type, int device, void* stream);

/* Overflow handling of the bucketing op (src/psh/batch_psh_bucket.cuh:154-246, 259-382).
 * 0 = hash + claim only (every point stays in its first-hash bucket);
 * 1 = deterministic probe rebalance + recycle (default). */
int f3d_set_psh_rebalance(int mode);
int f3d_get_psh_rebalance(void);

/* Rounding of the voxel quantiser's quotient (src/psh/hash_fns.cuh:23-33: (c - min) * num_vox / (max - min) in fp32),
 * for the bucketing op and the sub-bucket builder alike.
 * 0 = multiply by the correctly rounded reciprocal of (max - min): the form a build of the reference with
 *     nvcc --use_fast_math (its CMakeLists.txt:49-52) evaluates (default);
 * 1 = IEEE fp32 division, as the source text reads (a reference build without fast-math).
 * The two differ by at most one cell, for under 1 % of all fp16 inputs. */
int f3d_set_quantiser(int mode);
int f3d_get_quantiser(void);

/* Whole-batch bounding box of fp16 coordinates (replaces the two torch.min/max passes of
 * flash3dxfmr/psh/psh_main.py:117-118).  bbox_min/max [3] fp16, written in place. */
int f3d_coord_bbox(const f3d_half_t* coord, uint32_t total_n, f3d_half_t* bbox_min, f3d_half_t* bbox_max,
                   int device, void* stream);

/* ---- sub-bucket pooling: batch_subbuck_reduce, src/f3d_frontend.cu:60-66,
 *      src/psh/batch_subbuck_pooling_dispatcher.cu:35-144 ---------------------------------------
 * scattered_coord [total_n,3] fp16; scattered_feat [total_n,feat_dim] bf16; subbuck_id [total_n] u32;
 * subbuck_off [total_n] u16; reduced_batch_sep [batch_size] u32 (input: cumsum of ceil(n_b/S));
 * reduced_coord [reduced_aligned_n,3] fp16; reduced_feat [reduced_aligned_n,feat_dim] bf16;
 * unpool_ind [reduced_n,subbuck_size] u32 prefilled with a value >= total_n ("empty slot").
 * hash_type is accepted and ignored, as in the reference (dispatcher :108-109).
 * Rows [reduced_n, reduced_aligned_n) of reduced_coord / reduced_feat are zero-filled. */
int f3d_batch_subbuck_reduce(const f3d_half_t* scattered_coord, const f3d_bf16_t* scattered_feat,
                             const uint32_t* batch_sep, uint32_t batch_size, uint32_t total_n,
                             uint32_t instance_max_n, uint32_t feat_dim, uint32_t subbuck_size,
                             uint32_t num_vox, const f3d_half_t* bbox_min, const f3d_half_t* bbox_max,
                             uint32_t* subbuck_id, uint16_t* subbuck_off, const uint32_t* reduced_batch_sep,
                             f3d_half_t* reduced_coord, f3d_bf16_t* reduced_feat, uint32_t reduced_aligned_n,
                             uint32_t* unpool_ind, uint32_t reduced_n, uint32_t hash_type, uint32_t red_op,
                             int device, void* stream);

/* The two halves of the op above, separately callable (kernels local_subbuck_ker and
 * reduce_feat_ker, src/psh/batch_psh_subbuck_reduce.cuh:104-298 and :300-359). */
int f3d_subbuck_build(const f3d_half_t* coord, const uint32_t* batch_sep, uint32_t batch_size,
                      uint32_t total_n, uint32_t instance_max_n, uint32_t subbuck_size, uint32_t num_vox,
                      uint32_t* subbuck_id, uint16_t* subbuck_off, const uint32_t* reduced_batch_sep,
                      f3d_half_t* reduced_coord, uint32_t reduced_aligned_n, uint32_t* unpool_ind,
                      uint32_t reduced_n, int device, void* stream);
int f3d_reduce_feat(const f3d_bf16_t* feat, uint32_t total_n, uint32_t feat_dim, const uint32_t* unpool_ind,
                    uint32_t reduced_n, uint32_t subbuck_size, uint32_t red_op, f3d_bf16_t* reduced_feat,
                    uint32_t reduced_aligned_n, int device, void* stream);

/* The feature reduce with the layer that follows it in the reference's pooling wrapper applied to every reduced row
 * before it is stored (flash3dxfmr/layers/hourglass.py:104-109: pooling -> norm -> activation), alignment rows
 * included, as the layer applied to the whole tensor would.  norm_mode 1: LayerNorm (gamma, beta bf16 [feat_dim], beta
 * may be NULL; eps; act must be F3D_ACT_NONE); norm_mode 2: act(x * scale + shift) with fp32 scale / shift [feat_dim] (an
 * eval-mode BatchNorm1d folded) and act in {NONE, GELU, SILU, RELU}.  feat_dim a multiple of 8 (LayerNorm: 8 times a
 * power of two, at most 512), all tensors 16-byte aligned; F3D_ERR_UNSUPPORTED otherwise. */
int f3d_reduce_feat_norm(const f3d_bf16_t* feat, uint32_t total_n, uint32_t feat_dim, const uint32_t* unpool_ind,
                         uint32_t reduced_n, uint32_t subbuck_size, uint32_t red_op, f3d_bf16_t* reduced_feat,
                         uint32_t reduced_aligned_n, uint32_t norm_mode, const f3d_bf16_t* gamma, const f3d_bf16_t* beta,
                         const float* scale, const float* shift, float eps, uint32_t act, int device, void* stream);

/* ---- additive unpool: additive_unpool_fwd, src/f3d_frontend.cu:99-101,
 *      src/psh/additive_unpool_dispatcher.cu:26-79 ----------------------------------------------
 * up[r,:] = bf16(float(down[i,:]) + float(res[r,:])) for r = unpool_ind[i,s] < up_n. */
int f3d_additive_unpool_fwd(const f3d_bf16_t* res_feat, const f3d_bf16_t* down_feat, f3d_bf16_t* up_add_feat,
                            const uint32_t* unpool_ind, uint32_t up_n, uint32_t down_n, uint32_t feat_dim,
                            uint32_t subbuck_size, int device, void* stream);

/* The same with both operands normalised on the way in: up[r,:] = bf16(norm_down(down[i,:]) + norm_res(res[r,:])), where
 * the reference's unpooling wrapper runs Linear -> norm -> activation on each branch before the op
 * (flash3dxfmr/layers/hourglass.py:152-159).  Modes, parameters and limits as for f3d_reduce_feat_norm; one mode and one
 * activation for both branches, parameters per branch. */
int f3d_additive_unpool_norm_fwd(const f3d_bf16_t* res_feat, const f3d_bf16_t* down_feat, f3d_bf16_t* up_add_feat,
                                 const uint32_t* unpool_ind, uint32_t up_n, uint32_t down_n, uint32_t feat_dim,
                                 uint32_t subbuck_size, uint32_t norm_mode, const f3d_bf16_t* res_gamma,
                                 const f3d_bf16_t* res_beta, const float* res_scale, const float* res_shift, float res_eps,
                                 const f3d_bf16_t* down_gamma, const f3d_bf16_t* down_beta, const float* down_scale,
                                 const float* down_shift, float down_eps, uint32_t act, int device, void* stream);

/* ---- PSH permutation index and feature scatter: completes batch_psh_cumsum_scatter_feat_index_postpad_ker,
 *      src/psh/batch_psh_bucket.cuh:617-753 (unfinished in the reference: it writes the index, :735, and the pad
 *      value total_N + 3, :678, and moves no feature) ------------------------------------------------------------
 * Runs after f3d_batch_psh_scatter_pad_hash on that call's bucket_id / bucket_offset / bucket_counter /
 * cumsum_counter / batch_sep.  scatter_idx_out2in[dst] = src for every input row, = total_n + 3 for the pad rows
 * [total_n, pad_to_n); with feat != NULL also scattered_feat[dst] = feat[src] (rows of row_bytes bytes, any even
 * size) and zero pad rows.  scatter_idx_out2in [pad_to_n]; feat [total_n] rows; scattered_feat [pad_to_n] rows. */
int f3d_psh_scatter_feat_index(const uint16_t* bucket_id, const uint32_t* bucket_offset,
                               const uint32_t* bucket_counter, const uint32_t* cumsum_counter,
                               const uint32_t* batch_sep, uint32_t batch_size, uint32_t total_n, uint32_t num_bucket,
                               const void* feat, uint32_t row_bytes, uint32_t* scatter_idx_out2in,
                               void* scattered_feat, uint32_t pad_to_n, int device, void* stream);

/* Row permutation by such an index (no counterpart in the reference, which never reaches this step; it is what
 * src/psh/batch_psh_bucket.cuh:617-753 prepares the index for).
 * gather != 0: out[r] = index[r] < n_other ? in[index[r]] : 0   for r < n_index  (in: n_other rows, out: n_index rows)
 * gather == 0: out[index[r]] = in[r] where index[r] < n_other   for r < n_index  (in: n_index rows, out: n_other rows;
 *              rows of out that no index names keep the caller's content).
 * With the out-to-in index, gather moves input-order rows to PSH order and the other direction restores the input
 * order; each is the other's gradient. */
int f3d_permute_rows(const uint32_t* index, const void* in, void* out, uint32_t n_index, uint32_t n_other,
                     uint32_t row_bytes, uint32_t gather, int device, void* stream);

/* ---- additive unpool backward: additive_unpool_bwd, src/f3d_frontend.cu:103-105, kernel
 *      src/psh/additive_unpool.cuh:90-137, dispatcher src/psh/additive_unpool_dispatcher.cu:81-134 ----
 * grad_res[r,:] = grad_up_added[r,:] for every r = unpool_ind[i,s] < up_n (rows no slot refers to keep the
 * caller's content); grad_down[i,:] = bf16(sum over the valid slots of row i, slot order, fp32).
 * grad_res, grad_up_added [up_n, feat_dim]; grad_down [>= down_n, feat_dim]; unpool_ind [down_n, subbuck_size]. */
int f3d_additive_unpool_bwd(f3d_bf16_t* grad_res, f3d_bf16_t* grad_down, const f3d_bf16_t* grad_up_added,
                            const uint32_t* unpool_ind, uint32_t up_n, uint32_t down_n, uint32_t feat_dim,
                            uint32_t subbuck_size, int device, void* stream);

/* ---- sub-bucket reduce backward: batch_subbuck_reduce_backward, src/f3d_frontend.cu:68-71, kernel
 *      src/psh/batch_psh_subbuck_reduce_bwd.cuh:39-126 ----------------------------------------------------
 * red_op 0 mean: bf16(grad / max(count,1)) to every valid slot; 1 sum: grad to every valid slot; 2 min / 3 max:
 * grad to the first slot holding the strict winner of input_feat, zero to the other valid slots.
 * Rows of grad_input_feat that no slot refers to keep the caller's content.
 * grad_red_feat [>= reduced_n, feat_dim]; input_feat, grad_input_feat [total_n, feat_dim]. */
int f3d_subbuck_reduce_bwd(const f3d_bf16_t* grad_red_feat, const f3d_bf16_t* input_feat, const uint32_t* unpool_ind,
                           f3d_bf16_t* grad_input_feat, uint32_t total_n, uint32_t reduced_n, uint32_t feat_dim,
                           uint32_t subbuck_size, uint32_t red_op, int device, void* stream);

/* ---- bucketed attention backward: buck_swin_bwd, declared src/f3d_frontend.cu:94-97, called from
 *      flash3dxfmr/layers/buck_swin.py:69-95 (kernel source absent from the reference) ------------
 * q,k,v [batch,seq_len,num_head,head_dim] bf16 with row stride qkv_row_stride (elements); o, d_o, dq, dk, dv dense
 * [batch,seq_len,num_head,head_dim] bf16; lse (from the forward), delta (output: rowsum(d_o * o))
 * [batch,seq_len,num_head] fp32.  Rows that no scope covers are not written.  kv_len (may be NULL)
 * [seq_len/bucket_size] i32 is the forward's extension: rows of a bucket at or past its valid length get zero
 * gradients and add nothing to the others (they must still hold finite numbers).  Supported: head_dim 16, 32, 64 or
 * 128, scopes of any number of buckets up to 4096 (the reference's test shapes, tests/test_attn_bwd.py: head_dim 64 and
 * 128, 32 buckets of 256 in one scope); other head sizes return F3D_ERR_UNSUPPORTED. */
int f3d_buck_swin_bwd(const f3d_bf16_t* q, const f3d_bf16_t* k, const f3d_bf16_t* v, uint32_t qkv_row_stride,
                      const f3d_bf16_t* o, const f3d_bf16_t* d_o, const float* lse, float* delta, f3d_bf16_t* dq,
                      f3d_bf16_t* dk, f3d_bf16_t* dv, const uint32_t* scope_buckets, uint32_t num_scope,
                      uint32_t scope_size, uint32_t bucket_size, uint32_t batch, uint32_t seq_len, uint32_t num_head,
                      uint32_t head_dim, const int32_t* kv_len, int device, void* stream);

/* The same with dq, dk, dv rows `grad_row_stride` elements apart (each still dense over num_head * head_dim), e.g. the
 * three thirds of one [batch, seq_len, 3 * num_head * head_dim] gradient of the qkv projection output, which spares
 * the concatenation that torch's autograd would otherwise make of three dense tensors. */
int f3d_buck_swin_bwd_strided(const f3d_bf16_t* q, const f3d_bf16_t* k, const f3d_bf16_t* v, uint32_t qkv_row_stride,
                              const f3d_bf16_t* o, const f3d_bf16_t* d_o, const float* lse, float* delta,
                              f3d_bf16_t* dq, f3d_bf16_t* dk, f3d_bf16_t* dv, uint32_t grad_row_stride,
                              const uint32_t* scope_buckets, uint32_t num_scope, uint32_t scope_size,
                              uint32_t bucket_size, uint32_t batch, uint32_t seq_len, uint32_t num_head,
                              uint32_t head_dim, const int32_t* kv_len, int device, void* stream);

/* ---- bucketed attention forward: buck_swin_fwd, declared src/f3d_frontend.cu:90-92, called from
 *      flash3dxfmr/layers/buck_swin.py:57 (kernel source absent from the reference) --------------
 * q,k,v,o [batch,seq_len,num_head,head_dim] bf16 contiguous; lse [batch,seq_len,num_head] fp32;
 * scope_buckets [num_scope,scope_size] u32; every scope attends within the union of its buckets
 * (rows [k*bucket_size,(k+1)*bucket_size)).  kv_len (may be NULL) [seq_len/bucket_size] i32 is an
 * extension: valid rows per bucket; masked query rows get o = 0, lse = 0. */
int f3d_buck_swin_fwd(const f3d_bf16_t* q, const f3d_bf16_t* k, const f3d_bf16_t* v, f3d_bf16_t* o, float* lse,
                      const uint32_t* scope_buckets, uint32_t num_scope, uint32_t scope_size,
                      uint32_t bucket_size, uint32_t batch, uint32_t seq_len, uint32_t num_head,
                      uint32_t head_dim, const int32_t* kv_len, int device, void* stream);

/* Strided variant: q/k/v rows are `qkv_row_stride` elements apart (e.g. the three thirds of one
 * [seq, 3*C] projection output), which removes the three .contiguous() copies of
 * flash3dxfmr/layers/buck_swin.py:187-190.  o is dense [batch,seq_len,num_head,head_dim]. */
int f3d_buck_swin_fwd_strided(const f3d_bf16_t* q, const f3d_bf16_t* k, const f3d_bf16_t* v,
                              uint32_t qkv_row_stride, f3d_bf16_t* o, float* lse,
                              const uint32_t* scope_buckets, uint32_t num_scope, uint32_t scope_size,
                              uint32_t bucket_size, uint32_t batch, uint32_t seq_len, uint32_t num_head,
                              uint32_t head_dim, const int32_t* kv_len, int device, void* stream);

/* ---- frozen weights (extension; the reference leaves its dense layers to torch / TransformerEngine) -----------
 * f3d_ln_linear_bf16, f3d_ln_mlp_swiglu_bf16 and f3d_linear_bf16 (long inner dimension) first prepare their weights
 * (LayerNorm folded into the weight and bias, fragment-major copies): one small launch per call, into the library's
 * workspace.  A caller whose weights do not change between calls (inference) stages a buffer of its own instead:
 * the NEXT dense call on this thread prepares into `buf` (device memory, 256-byte aligned, `bytes` long; for a
 * weight of n rows and k columns 3 n k + 4 n + 2 k + 512 bytes cover every case, with n = the fc1 rows for the
 * gated MLP), or, with ready != 0, takes what an earlier call with the same weights and shapes left there and skips
 * the preparation launch.  The staging ends with that call whatever its outcome.  A buffer that is too small makes
 * the call fail with a message. */
int f3d_stage_weights(void* buf, size_t bytes, int ready);

/* ---- dense layers --------------------------------------------------------------------------
 * gemm_sm_bf16(A[M,K], B[K,N], O[M,N]) — src/f3d_frontend.cu:87-88, src/psh/gemm_dispatcher.cu;
 * the reference only accepts M == 128, this one any shape with K % 8 == 0 and N % 8 == 0. */
int f3d_gemm_sm_bf16(const f3d_bf16_t* a, const f3d_bf16_t* b, f3d_bf16_t* o, uint32_t m, uint32_t n,
                     uint32_t k, int device, void* stream);

/* y = act(x · wᵀ + bias) + residual — the nn.Linear / te.Linear sites of the layer API
 * (flash3dxfmr/layers/buck_swin.py:159,163; hourglass.py:65,148,150; flash3d.py:32).
 * x [m,k] bf16 (row stride ldx), w [n,k] bf16, bias [n] bf16 or NULL, residual [m,n_out] bf16 or
 * NULL (row stride ldr), y [m,n_out] bf16 (row stride ldy); n_out = n/2 for F3D_ACT_SWIGLU else n.
 * fp32 accumulate; k % 8 == 0. */
int f3d_linear_bf16(const f3d_bf16_t* x, uint32_t ldx, const f3d_bf16_t* w, const f3d_bf16_t* bias,
                    const f3d_bf16_t* residual, uint32_t ldr, f3d_bf16_t* y, uint32_t ldy, uint32_t m,
                    uint32_t n, uint32_t k, uint32_t act, int device, void* stream);

/* LayerNorm fused into the following linear layer: y = act(LayerNorm(x; gamma, beta, eps) · wᵀ + bias)
 * + residual, the `norm -> qkv` and `LayerNormMLP` front halves of flash3dxfmr/layers/stage.py:94-99.
 * Same tensor contract as f3d_linear_bf16 with k in {32, 64, 128, 256, 512}; gamma [k] bf16, beta [k]
 * bf16 or NULL.  LayerNorm is applied algebraically (w scaled by gamma and rounded to bf16, the row
 * statistics applied to the fp32 accumulators), so roundings fall in other places than in a separate
 * LayerNorm module followed by a Linear; the result is as close to the unrounded mathematics. */
int f3d_ln_linear_bf16(const f3d_bf16_t* x, uint32_t ldx, const f3d_bf16_t* gamma, const f3d_bf16_t* beta, float eps,
                       const f3d_bf16_t* w, const f3d_bf16_t* bias, const f3d_bf16_t* residual, uint32_t ldr,
                       f3d_bf16_t* y, uint32_t ldy, uint32_t m, uint32_t n, uint32_t k, uint32_t act, int device,
                       void* stream);

/* The whole gated MLP of a block in one kernel:
 *   y = (silu(LN(x) w1[:h]ᵀ + b1[:h]) * (LN(x) w1[h:]ᵀ + b1[h:])) w2ᵀ + b2 (+ residual),
 * te.LayerNormMLP(activation = "swiglu") followed by the residual add (flash3dxfmr/layers/elem_wise.py:22-26,
 * stage.py:94-97).  x [m,c] (row stride ldx), gamma [c], beta [c] or NULL, w1 [2 hidden, c] (value rows, then gate
 * rows), b1 [2 hidden] or NULL, w2 [c, hidden], b2 [c] or NULL, residual [m,c] or NULL (row stride ldr), y [m,c] (row
 * stride ldy), all bf16.  The hidden activations are rounded to bf16 as a separate fc1 kernel would store them and
 * never leave the registers.  c in {128, 256} with hidden a multiple of 32 (weights stream through LDS), or c in
 * {32, 64} with hidden a multiple of 32 up to 640 / 288 (all weights resident in LDS, each wave walks row tiles on its
 * own); anything else returns F3D_ERR_UNSUPPORTED without touching y (use f3d_ln_linear_bf16 with F3D_ACT_SWIGLU followed by f3d_linear_bf16).  Uses the per-device
 * workspace like f3d_ln_linear_bf16. */
int f3d_ln_mlp_swiglu_bf16(const f3d_bf16_t* x, uint32_t ldx, const f3d_bf16_t* gamma, const f3d_bf16_t* beta, float eps,
                           const f3d_bf16_t* w1, const f3d_bf16_t* b1, const f3d_bf16_t* w2, const f3d_bf16_t* b2,
                           const f3d_bf16_t* residual, uint32_t ldr, f3d_bf16_t* y, uint32_t ldy, uint32_t m,
                           uint32_t c, uint32_t hidden, int device, void* stream);

/* The second half of a transformer block in one kernel (flash3dxfmr/layers/stage.py:92-102: `proj`, the residual
 * add, then the MLP with its residual):
 *   x1 = a w_projT + b_proj + x,   y = x1 + MLP(LayerNorm(x1))   with the MLP of f3d_ln_mlp_swiglu_bf16.
 * a [m,c] (row stride lda) is the attention output, x [m,c] (row stride ldx) the block input, w_proj [c,c], b_proj [c]
 * or NULL; the other arguments as in f3d_ln_mlp_swiglu_bf16 (no residual argument: x1 is the residual).  x1 is rounded
 * to bf16 once, from the fp32 sum, and is held in registers only.  c in {128, 256} with hidden a multiple of 32, or
 * c in {32, 64} while all weights fit into LDS (as for f3d_ln_mlp_swiglu_bf16, with c * c * 2 bytes more); anything else
 * returns F3D_ERR_UNSUPPORTED without touching y (use f3d_linear_bf16 with the residual,
 * then f3d_ln_mlp_swiglu_bf16).  Inference only: no backward consumes its result. */
int f3d_proj_ln_mlp_swiglu_bf16(const f3d_bf16_t* a, uint32_t lda, const f3d_bf16_t* w_proj, const f3d_bf16_t* b_proj,
                                const f3d_bf16_t* x, uint32_t ldx, const f3d_bf16_t* gamma, const f3d_bf16_t* beta, float eps,
                                const f3d_bf16_t* w1, const f3d_bf16_t* b1, const f3d_bf16_t* w2, const f3d_bf16_t* b2,
                                f3d_bf16_t* y, uint32_t ldy, uint32_t m, uint32_t c, uint32_t hidden, int device,
                                void* stream);

/* The same with the block input formed inside the kernel from the points' coordinates: x = embed(coord), the
 * `PSH3DCoordEmbedding` output that feeds the FIRST block (flash3dxfmr/layers/psh_ops.py:64-68), never stored.  coord [m,3]
 * fp16 and embed_table [c,8] bf16 as in f3d_embed_ln_linear_bf16; the embedding enters the sum in fp32 (one product per 32
 * channels on the matrix core), x1 is rounded to bf16 once.  Same widths and return codes as
 * f3d_proj_ln_mlp_swiglu_bf16. */
int f3d_embed_proj_ln_mlp_swiglu_bf16(const f3d_bf16_t* a, uint32_t lda, const f3d_bf16_t* w_proj, const f3d_bf16_t* b_proj,
                                      const f3d_half_t* coord, const f3d_bf16_t* embed_table, const f3d_bf16_t* gamma,
                                      const f3d_bf16_t* beta, float eps, const f3d_bf16_t* w1, const f3d_bf16_t* b1,
                                      const f3d_bf16_t* w2, const f3d_bf16_t* b2, f3d_bf16_t* y, uint32_t ldy, uint32_t m,
                                      uint32_t c, uint32_t hidden, int device, void* stream);

/* The first block's `norm -> qkv -> attention` (flash3dxfmr/layers/stage.py:94-96, buck_swin.py:176-192) on the
 * coordinate embedding (psh_ops.py:64-68) without embedding, LayerNorm output or projection output ever being stored
 * (extension; inference only).  The embedding is x = E c with c = (x, y, z, 1) and E = [w_embed | b_embed]; over the
 * channels x - mean(x) = E' c (E' = E minus its column means) and var(x) = |L c|^2 (L: upper Cholesky factor of
 * E'^T E' / C), hence   qkv = rstd (M c) + b',  M = w_qkv diag(gamma) E',  b' = w_qkv beta + b_qkv,  rstd = 1 / sqrt(|L c|^2 + eps):
 * four multiplications per output instead of C, exact in real arithmetic (the embedding and the LayerNorm output are
 * not rounded to bf16 in between, so the result is closer to the unrounded mathematics than the three stored steps).
 *
 * f3d_embed_qkv_fold_bf16 prepares, from embed_w [c,3], embed_b [c] or NULL, gamma [c] or NULL, beta [c] or NULL, w_qkv [3c,c], b_qkv [3c]
 * or NULL (all bf16): `table` [num_head][4][32][16] bf16 (per head: Q in units of log2(e)/sqrt(head_dim), K, V, Q unscaled;
 * each number as a bf16 high and low part) and `chol` [16] fp32 (the ten entries of L row by row, eps, zeros).  Once per
 * set of weights.  head_dim must be 32 (F3D_ERR_UNSUPPORTED otherwise).
 *
 * f3d_embed_buck_swin_fwd is f3d_buck_swin_fwd with Q, K, V formed inside the kernel: a wave builds its 32 rows of an
 * item from their coordinates (coord [batch * seq_len, 3] fp16, the scattered coordinates) with three products on the
 * matrix core and writes K and V straight into LDS.  o, lse, scope_buckets and the sizes as in f3d_buck_swin_fwd; no
 * valid lengths.  head_dim 32 with scopes of 256 or 512 tokens; anything else returns F3D_ERR_UNSUPPORTED without
 * touching o (use f3d_embed_ln_linear_bf16, then f3d_buck_swin_fwd_strided). */
int f3d_embed_qkv_fold_bf16(const f3d_bf16_t* embed_w, const f3d_bf16_t* embed_b, const f3d_bf16_t* gamma,
                            const f3d_bf16_t* beta, float eps, const f3d_bf16_t* w_qkv, const f3d_bf16_t* b_qkv, uint32_t c,
                            uint32_t num_head, uint32_t head_dim, f3d_bf16_t* table, float* chol, int device,
                            void* stream);
int f3d_embed_buck_swin_fwd(const f3d_half_t* coord, const f3d_bf16_t* table, const float* chol, f3d_bf16_t* o, float* lse,
                            const uint32_t* scope_buckets, uint32_t num_scope, uint32_t scope_size, uint32_t bucket_size,
                            uint32_t batch, uint32_t seq_len, uint32_t num_head, uint32_t head_dim, int device,
                            void* stream);

/* LayerNorm over the last axis, fp32 statistics (norm callables of flash3dxfmr/layers/stage.py:67).
 * x,y [m,c] bf16; gamma,beta [c] bf16 (beta may be NULL). */
int f3d_layernorm_bf16(const f3d_bf16_t* x, const f3d_bf16_t* gamma, const f3d_bf16_t* beta, f3d_bf16_t* y,
                       uint32_t m, uint32_t c, float eps, int device, void* stream);

/* Coordinate embedding input cast + K=3 linear of PSH3DCoordEmbedding
 * (flash3dxfmr/layers/psh_ops.py:64-67): y[r,:] = bf16(coord[r,:]) · wᵀ + bias; w [c,3] bf16. */
int f3d_coord_embed_bf16(const f3d_half_t* coord, const f3d_bf16_t* w, const f3d_bf16_t* bias, f3d_bf16_t* y,
                         uint32_t m, uint32_t c, int device, void* stream);

/* The coordinate embedding fused into its first consumer (extension): y = LayerNorm(embed(coord)) wT + bias without
 * the embedding ever being stored, the `PSH3DCoordEmbedding` output feeding `norm -> qkv` of the first block
 * (flash3dxfmr/layers/psh_ops.py:64-68, stage.py:94-96).  coord [m,3] fp16 (the scattered coordinates); embed_table
 * [k,8] bf16 holds (w[c,0], w[c,1], w[c,2], bias[c], 0, 0, 0, 0) per embedding channel c; gamma, beta, eps, w [n,k],
 * bias [n] or NULL, y [m,n] (row stride ldy) as in f3d_ln_linear_bf16.  The kernel forms each row's embedding on the
 * matrix core (fp32 sum of the three products and the bias, rounded to bf16 as the embedding layer stores it) and goes
 * on as f3d_ln_linear_bf16.  k in {32, 64, 128, 256}, n a multiple of 32; anything else returns F3D_ERR_UNSUPPORTED
 * without touching y (use f3d_coord_embed_bf16, then f3d_ln_linear_bf16). */
int f3d_embed_ln_linear_bf16(const f3d_half_t* coord, const f3d_bf16_t* embed_table, const f3d_bf16_t* gamma,
                             const f3d_bf16_t* beta, float eps, const f3d_bf16_t* w, const f3d_bf16_t* bias, f3d_bf16_t* y,
                             uint32_t ldy, uint32_t m, uint32_t n, uint32_t k, int device, void* stream);

/* Per-channel affine + optional activation: eval-mode BatchNorm1d folded to scale/shift followed
 * by GELU/ReLU (pool / unpool norm+act callables, tests/test_psh_hourglass.py:103-106).
 * y = act(x * scale + shift); x,y [m,c] bf16; scale,shift [c] fp32. */
int f3d_affine_act_bf16(const f3d_bf16_t* x, const float* scale, const float* shift, f3d_bf16_t* y, uint32_t m,
                        uint32_t c, uint32_t act, int device, void* stream);

/* ---- backward of the dense layers ---------------------------------------------------------------
 * The reference takes these from torch / TransformerEngine autograd (flash3dxfmr/layers/buck_swin.py:159-163,
 * elem_wise.py:22-26, stage.py:94-99: nn.Linear, te.LayerNormMLP, the norms); the input gradient of a linear layer is
 * f3d_linear_bf16 with the transposed weight (dx = dy · w).
 *
 * Weight and bias gradient of y = x · wᵀ + b:  dw[n,k] = sum_m dy[m,n] x[m,k],  db[n] = sum_m dy[m,n].
 * dy [m,n] bf16 (row stride lddy), x [m,k] bf16 (row stride ldx), dw [n,k] fp32, db [n] fp32 or NULL; n % 8 == 0,
 * k % 8 == 0; fp32 accumulation in a fixed order (bit-reproducible).  accumulate != 0 adds to dw / db.  Uses the
 * per-device workspace like f3d_ln_linear_bf16. */
int f3d_linear_wgrad_bf16(const f3d_bf16_t* dy, uint32_t lddy, const f3d_bf16_t* x, uint32_t ldx, float* dw, float* db,
                          uint32_t m, uint32_t n, uint32_t k, uint32_t accumulate, int device, void* stream);

/* LayerNorm backward: with xhat = (x - mean) rstd and g = dh * gamma,
 *   dx = rstd (g - mean(g) - xhat mean(g xhat)) (+ dres),  dgamma = sum_rows dh xhat,  dbeta = sum_rows dh.
 * x, dh, dx [m,c] bf16 (row strides ldx, lddh, lddx), gamma [c] bf16, dres [m,c] bf16 or NULL (a gradient that
 * reaches x by another route, e.g. the residual connection; row stride lddr), dgamma, dbeta [c] fp32 (accumulate != 0
 * adds to them).  c in {32, 64, 128, 256, 512}, else F3D_ERR_UNSUPPORTED.  dx may alias dh or dres.  Uses the
 * per-device workspace. */
int f3d_layernorm_bwd_bf16(const f3d_bf16_t* x, uint32_t ldx, const f3d_bf16_t* dh, uint32_t lddh,
                           const f3d_bf16_t* gamma, const f3d_bf16_t* dres, uint32_t lddr, f3d_bf16_t* dx, uint32_t lddx,
                           float* dgamma, float* dbeta, uint32_t m, uint32_t c, float eps, uint32_t accumulate,
                           int device, void* stream);

/* Backward of the gated activation a = silu(z[:, :h]) * z[:, h:] (F3D_ACT_SWIGLU):
 *   dz[:, :h] = da * z2 * s (1 + z1 (1 - s)),  dz[:, h:] = da * silu(z1),  s = sigmoid(z1).
 * z, dz [m,2h] bf16, da [m,h] bf16, a [m,h] bf16 or NULL (the recomputed activation, which the weight gradient of
 * the following layer needs).  dz may alias z and a may alias da. */
int f3d_swiglu_bwd_bf16(const f3d_bf16_t* z, uint32_t ldz, const f3d_bf16_t* da, uint32_t ldda, f3d_bf16_t* dz,
                        uint32_t lddz, f3d_bf16_t* a, uint32_t lda, uint32_t m, uint32_t hidden, int device,
                        void* stream);

/* The middle of the gated MLP's backward in one kernel: with h = LayerNorm(x) [m,c], dy [m,c], w1 [2 hidden, c] (value
 * rows, then gate rows), b1 [2 hidden] or NULL and w2t = w2 transposed [hidden, c], it recomputes [z1 | z2] = h · w1ᵀ + b1,
 * forms da = dy · w2 and writes a = silu(z1) * z2 [m,hidden] and dz [m, 2 hidden] (as f3d_swiglu_bwd_bf16 defines them);
 * neither z nor da is stored.  c in {32, 64, 128, 256}, hidden a multiple of 32, else F3D_ERR_UNSUPPORTED (then: f3d_linear_bf16
 * twice and f3d_swiglu_bwd_bf16). */
int f3d_mlp_gate_bwd_bf16(const f3d_bf16_t* h, uint32_t ldh, const f3d_bf16_t* dy, uint32_t lddy, const f3d_bf16_t* w1,
                          const f3d_bf16_t* b1, const f3d_bf16_t* w2t, f3d_bf16_t* dz, uint32_t lddz, f3d_bf16_t* a,
                          uint32_t lda, uint32_t m, uint32_t c, uint32_t hidden, int device, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* F3D_HIP_H */
