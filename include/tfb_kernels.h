/* C-ABI of libtfb_hip.so: hand-written HIP kernels for gfx950 (MI355X) that replace the NKI kernels on the
 * training-step hot path of Danishlynx/trainium-frontier-them-bones.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless the comment says "host"; bf16 tensors are raw 16-bit words,
 *     fp8 tensors raw bytes (OCP e4m3fn / e5m2), row-major, contiguous unless strides are passed;
 *   - `stream` is a hipStream_t; kernels are launched on it and the call returns without synchronising;
 *   - no entry point allocates, frees or synchronises; scratch and workspaces are caller-owned (one exception:
 *     tfb_attn_bwd_static keeps its scratch in a static device array of the library);
 *   - return value: 0 ok, 1 unsupported shape (the reference wrappers' "shapes_apply() is false": the caller runs
 *     its own fallback or raises), 2 bad argument, 3 launch failed, 4 workspace too small.
 *
 * Each declaration cites the reference interface it replaces (paths relative to the reference repository).
 */
#ifndef TFB_KERNELS_H
#define TFB_KERNELS_H

#ifdef __cplusplus
extern "C" {
#endif

/* ---- bf16 GEMM ------------------------------------------------------------------------------------------------
 * C[M,N] (+)= op(A) @ op(B); A is [M,K] (trans_a=0) or [K,M]; B is [K,N] (trans_b=0) or [N,K]; fp32 accumulation;
 * C bf16 (out_f32=0) or fp32; accumulate=1 adds into C (one rounding). M, N multiples of 128, K of 64.
 * workspace: optional fp32 split-K scratch (used when the output has few tiles and K is long).
 * Replaces nki_matmul(a, b, trans_a, trans_b): round1/source/train.py:1137 (kernels 926, 1052) and the in-place
 * weight-gradient accumulate of round1/source/train.py:8463-8509. */
int tfb_gemm_bf16(const void* A, const void* B, void* C, int M, int N, int K, int trans_a, int trans_b, int out_f32,
                  int accumulate, void* workspace, long workspace_bytes, void* stream);
/* tfb_gemm_bf16 with the product multiplied by the device fp32 scalar *alpha (NULL = 1) before its one rounding:
 * C (+)= alpha op(A) @ op(B). The gradient GEMMs of the LM head take the loss's upstream gradient this way
 * (autograd's grad_output of round1/source/train.py:9191-9212's loss, which the reference multiplies into dlogits). */
int tfb_gemm_bf16_scaled(const void* A, const void* B, void* C, int M, int N, int K, int trans_a, int trans_b, int out_f32,
                         int accumulate, void* workspace, long workspace_bytes, const void* alpha, void* stream);
/* C [M,N] = bf16(res + bf16(A [M,K] @ op(B))), res [M,N] bf16: a projection with the residual add that follows it made in
 * the GEMM's store; equal to tfb_gemm_bf16 followed by a bf16 add, bit for bit. B is [K,N] (trans_b=0) or [N,K].
 * The bf16 form of _proj8_fwd_ra_kernel (round2/source/kernels/nki_attn_nr8.py:1003: out = bf16(res + bf16(acc dq))). */
int tfb_gemm_bf16_res(const void* A, const void* B, const void* res, void* C, int M, int N, int K, int trans_b, void* stream);

/* ---- RMSNorm family --------------------------------------------------------------------------------------------
 * Number of partial-sum rows the backward kernels write for `nrows` rows (host helper, no GPU work). */
int tfb_norm_bwd_blocks(long nrows);

/* s = x (res NULL) or bf16(x + res) written to s_out; y = bf16(s * rsqrt(mean(s^2) + eps) * w) (w NULL = no weight);
 * inv fp32 [nrows] = the rsqrt factor. C multiple of 8, <= 4096.
 * Replaces rmsnorm_fast (round1/source/train.py:5594, kernels 5378), tail_norm2 (6117, kernel 5887), final_norm
 * (6826) and nf_norm_rows (round2/source/train.py:8805). */
int tfb_rmsnorm_fwd(const void* x, const void* res, const void* w, void* s_out, void* y, void* inv, long nrows, int C,
                    float eps, void* stream);
/* tfb_rmsnorm_fwd that also writes y8 [nrows][C] = e4m3(bf16(y) * y8_scale): the operand cast of the fp8 GEMM that
 * consumes y (tfb_mlp8_fwd's x8 at the constant scale 4, tfb_gemm_fp8's a8), made in the norm's pass instead of one of
 * its own. Replaces the norm prologue of _mlp8_fwd_nr_kernel (round2/source/kernels/nki_mlp_nr8.py:1032: xn, rs and the
 * casts at X_SCALE) and of _proj8_fwd_nm_kernel (round2/source/kernels/nki_attn_nr8.py:929). y may be NULL here: with the
 * weight gradients in fp8 too nothing reads the bf16 rows, and they are then not written. */
int tfb_rmsnorm_fwd_q(const void* x, const void* res, const void* w, void* s_out, void* y, void* inv, void* y8,
                      float y8_scale, long nrows, int C, float eps, void* stream);

/* dx = gs + inv * (gh - s * (gh . s) * inv^2 / C), gh = gy * w; dw fp32 [C] (+)= sum_rows gy * s * inv.
 * dw_part: fp32 [tfb_norm_bwd_blocks(nrows)][C] scratch (needed only with w).
 * Replaces _rms_bwd_kernel / _tail_bwd (round1/source/train.py:5410, 5927) and nf_norm_backward
 * (round2/source/train.py:8813-8825). */
int tfb_rmsnorm_bwd(const void* gy, const void* gs, const void* s, const void* w, const void* inv, void* dx, void* dw_part,
                    void* dw, int dw_accumulate, long nrows, int C, void* stream);

/* tfb_rmsnorm_bwd that also leaves amax_part fp32 [tfb_norm_bwd_blocks(nrows)]: per workgroup, the largest |dx| it wrote
 * (of the rounded values), for the fp8 MLP whose backward receives this dx as its dy (tfb_mlp8_backward_scales_part).
 * Has no counterpart in the reference, whose backward_scales reads dy for its amax (nki_mlp_fused8.py:803). */
int tfb_rmsnorm_bwd_amax(const void* gy, const void* gs, const void* s, const void* w, const void* inv, void* dx, void* dw_part,
                         void* dw, int dw_accumulate, void* amax_part, long nrows, int C, void* stream);

/* tfb_rmsnorm_bwd with dw = NULL leaves the weight gradient as per-workgroup partial sums in dw_part; this call finishes
 * `count` of them in one launch: dw[i][c] (+)= sum_r dw_part[i][r][c], i < count, r < tfb_norm_bwd_blocks(nrows)
 * (part_stride, dw_stride: floats between consecutive i). The sums are taken in a fixed order (bit-reproducible).
 * Has no counterpart in the reference, whose wrappers finish each gain gradient with a torch .sum
 * (round1/source/train.py:6039); it exists because 25 separate 12-workgroup reductions cost 0.5 ms of the step. */
int tfb_norm_dw_finish(const void* dw_part, void* dw, int count, long part_stride, long dw_stride, int dw_accumulate,
                       long nrows, int C, void* stream);

/* x_new = bf16(l1 (x [+ l3 skip]) + l2 x0); x_norm = RMSNorm(x_new); gains = fp32 [3] device (l1, l2, l3).
 * Replaces block_head (round1/source/train.py:5578, kernel 5257) and head_skip (6106, kernel 5743). */
int tfb_block_head_fwd(const void* x, const void* x0, const void* skip, const void* gains, void* x_new, void* x_norm,
                       void* inv, long nrows, int C, float eps, void* stream);

/* G = g_new + J^T(g_norm); dx = l1 G, dx0 = l2 G, dskip = l3 G; dgains fp32 [4] = (sum G.x, sum G.x0, sum G.skip, 0).
 * gain_part: fp32 [tfb_norm_bwd_blocks(nrows)][4] scratch.
 * Replaces _bh_bwd_kernel / _hs_bwd (round1/source/train.py:5301, 5793). */
int tfb_block_head_bwd(const void* g_new, const void* g_norm, const void* x, const void* x0, const void* skip,
                       const void* x_new, const void* inv, const void* gains, void* dx, void* dx0, void* dskip,
                       void* gain_part, void* dgains, long nrows, int C, void* stream);

/* ---- elementwise ------------------------------------------------------------------------------------------------
 * mode 0: out = relu(a)^2; mode 1: out = b * 2 relu(a) (a = x, b = gy); mode 2: out = bf16(sqrt(4 a)) * b (a = h).
 * Replaces relu_squared / relu2_backward / relu2_backward_from_h (round1/source/train.py:663, 597, 633). */
int tfb_relu2(const void* a, const void* b, void* out, long n, int mode, void* stream);

/* Half-split rotation of `nheads` heads of D columns at the start of each row (row r = token r % T); cos/sin bf16
 * [T][D/2]; inverse=1 applies the transpose rotation (the backward). In place when out == x.
 * Replaces the RoPE step of round1/source/train.py:4188-4193 (rope_norm 4447 without its QK-norm). */
int tfb_rope(const void* x, const void* cos_t, const void* sin_t, void* out, long rows, int T, int nheads, int D,
             long row_stride, long out_stride, int inverse, void* stream);

/* RoPE followed by the parameter-free RMSNorm of every head (the attention block's QK-norm): r = bf16(rope(x)) (NULL to
 * skip), inv [rows][nheads] fp32 = rsqrt(mean_D(r^2) + eps), y = bf16(r inv). Head layout as tfb_rope; D = 64 or 128;
 * strides in elements (multiples of 8). Replaces rope_norm(x, cos, sin) (round1/source/train.py:4447; eager form 4184-4196)
 * and the rotation + QK-norm prologue of nki_rope_attention (round1/source/train.py:8197; r5 / inv3 of
 * round2/source/kernels/nki_attn_bandpro.py:1850). */
int tfb_rope_norm_fwd(const void* x, const void* cos_t, const void* sin_t, void* r, void* y, void* inv, long rows, int T,
                      int nheads, int D, long x_stride, long r_stride, long y_stride, float eps, void* stream);

/* dx = the gradient of tfb_rope_norm_fwd's input: dr = bf16(inv (g - rh (g . rh) / D)), rh = r inv, then the transposed
 * rotation. dx may alias g. Replaces the backward of rope_norm (round1/source/train.py:4339 _rope_norm_bwd_kernel; forward kernel 4308). */
int tfb_rope_norm_bwd(const void* g, const void* r, const void* inv, const void* cos_t, const void* sin_t, void* dx, long rows,
                      int T, int nheads, int D, long g_stride, long r_stride, long dx_stride, void* stream);

int tfb_resmix_bwd_blocks(long n);
/* dx = g bf16(a), dx0 = g bf16(b), dab fp32 [2] = (sum bf16(g x), sum bf16(g x0)); ab fp32 [2] device;
 * part: fp32 [2 * tfb_resmix_bwd_blocks(n)] scratch.
 * Replaces _resmix_bwd_kernel (round2/source/kernels/nki_resmix.py; emulate :148-162). */
int tfb_resmix_bwd(const void* g, const void* x, const void* x0, const void* ab, void* dx, void* dx0, void* part, void* dab,
                   long n, void* stream);

/* out[i] = w[idx[i]] rows, w [V][C]; idx int64 (idx64=1) or int32. An id outside [0, V) is never used as an address: its
 * output row is zeros, and the backward calls below give it no gradient. Replaces embedding_fwd
 * (round1/source/train.py:8407). */
int tfb_embedding_fwd(const void* idx, int idx64, const void* w, void* out, long n, int C, int V, void* stream);
/* dw_f32[idx[i]] += dy[i] (fp32 atomics), dw_f32 [V][C]. Replaces _emb_bwd_kernel (round1/source/train.py:8303). */
int tfb_embedding_bwd(const void* idx, int idx64, const void* dy, void* dw_f32, long n, int C, int V, void* stream);
/* The same sum with the rows grouped by token first (counting sort on the device, then a segmented sum), so that the
 * frequent tokens of a Zipf batch do not serialize on atomics; ids outside [0, V) are dropped. scratch: int32
 * [tfb_embedding_bwd_scratch_ints(n, V)]. Replaces _emb_bwd_kernel (round1/source/train.py:8303). */
long tfb_embedding_bwd_scratch_ints(long n, int V);
int tfb_embedding_bwd_grouped(const void* idx, int idx64, const void* dy, void* dw_f32, long n, int C, int V, void* scratch,
                              void* stream);

/* One AdamW update in place on fp32 p, m, v from g (fp32 if g_f32 else bf16); optional bf16 copy of p.
 * p *= 1 - lr wd; m = lerp(m, g, 1-b1); v = lerp(v, g^2, 1-b2); p -= lr (m / bias1) / (sqrt(v / bias2) + eps).
 * Replaces adamw_fused_step (round1/source/train.py:1573, kernel 1410; math 9670-9677). */
int tfb_adamw(void* p, const void* g, int g_f32, void* m, void* v, void* p_bf16, long n, float lr, float wd,
              float one_minus_beta1, float one_minus_beta2, float eps, float bias1, float bias2, void* stream);

/* p[0..n) = val with a kernel (safe inside HIP graph capture, unlike a memset node). No reference counterpart. */
int tfb_fill_f32(void* p, float val, long n, void* stream);

/* ---- fp8 fused MLP ------------------------------------------------------------------------------------------------
 * fp32 scratch elements tfb_mlp8_forward_scales needs (host helper). */
long tfb_mlp8_scale_scratch_floats(int F);

/* row_out fp32 [16] = the layer's scale row from w_fc [F][d], w_proj [d][F] (bf16): columns s_wfc, dq_fc, c_h, s_wproj,
 * dq_proj, s_dy, dq_dh2, s_dp, dq_dx, rho2, kappa2, i_wfc, i_wproj, s_h, amax_wfc, amax_wproj.
 * Replaces forward_scales (round2/source/kernels/nki_mlp_fused8.py:782-800) and the statistics kernels of
 * round2/source/kernels/nki_scstat.py. e4m3_limit 240 gives the reference's rows. x_scale: the activation scale the
 * forward casts x at (the reference's constant 4), or x_scale_dev (not NULL: a device fp32 scalar, e.g. tfb_amax_scale's
 * output, read by the kernel so that a per-tensor amax scale costs no host synchronisation; x_scale is then ignored). */
int tfb_mlp8_forward_scales(const void* w_fc, const void* w_proj, void* row_out, void* scratch, int F, int d,
                            float e4m3_limit, float x_scale, const void* x_scale_dev, void* stream);

/* row_out = row_in with s_dy, dq_dh2, s_dp, dq_dx filled from amax(dy); scratch fp32 [1024].
 * Replaces backward_scales (nki_mlp_fused8.py:803-813). */
int tfb_mlp8_backward_scales(const void* dy, const void* row_in, void* row_out, void* scratch, long M, int d, void* stream);
/* The same row from npart amax partials whose maximum is amax(dy) (as tfb_rmsnorm_bwd_amax leaves them): no pass over dy.
 * Replaces backward_scales (nki_mlp_fused8.py:803-813). */
int tfb_mlp8_backward_scales_part(const void* amax_part, int npart, const void* row_in, void* row_out, int d, void* stream);

/* out fp32 [3] = (s, 1/s, amax): s = 2^e the largest with amax(x) s <= limit, e in [e_lo, e_hi]; scratch fp32 [1024].
 * The reference's _pow2_le (nki_mlp_fused8.py:742) applied to a tensor's amax. */
int tfb_amax_scale(const void* x, long n, float limit, int e_lo, int e_hi, void* out, void* scratch, void* stream);

/* out8 = fp8(x * scale): scale read from scale_ptr (device fp32) when non-NULL, else scale_imm. fmt 0 e4m3, 1 e5m2.
 * The reference's q8 (nki_mlp_fused8.py:821-825) producing bytes. */
int tfb_quant_fp8(const void* x, const void* scale_ptr, float scale_imm, int fmt, void* out8, long n, void* stream);

/* w8 uint8 [4][F*d] = e4m3(w_fc s_wfc) as [F][d] and [d][F], e4m3(w_proj s_wproj) as [d][F] and [F][d].
 * Replaces _precast8_kernel / precast_ref (round2/source/kernels/nki_mlp_l4t.py:392, 948-970). */
int tfb_mlp8_precast(const void* w_fc, const void* w_proj, const void* row, void* w8, int F, int d, void* stream);

/* tfb_mlp8_forward_scales + tfb_mlp8_precast for `layers` MLPs in four launches: rows fp32 [layers][16], w8 uint8
 * [layers][4][F*d], from weights laid out with one stride (layer i's w_fc at w_fc + i * layer_stride elements, its
 * w_proj at w_proj + i * layer_stride). scratch: layers * tfb_mlp8_scale_scratch_floats(F) floats. F, d multiples of 64.
 * Replaces the loop over layers of fp8_refresh_weights (round2/source/train.py:6617: mlp8_scales_into 7003 +
 * mlp8_precast_into 7267 per layer). */
int tfb_mlp8_refresh_layers(const void* w_fc, const void* w_proj, long layer_stride, int layers, void* rows, void* w8,
                            void* scratch, int F, int d, float e4m3_limit, float x_scale, void* stream);

/* Forward from x8 = e4m3(x s_x) [M][d]: y bf16 [M][d], r bf16 [M][F] (saved for backward), h8 [M][F] byte scratch.
 * M % 128 == 0, d % 256 == 0, F % 256 == 0 (the reference's shapes_apply8, nki_mlp_fused8.py:666).
 * Replaces _mlp8_fwd_kernel / _mlp8_fwd_pc_kernel (nki_mlp_fused8.py:509, nki_mlp_l4t.py:434); op s2mlp8::fwd
 * (round2/source/train.py:6858). r is token-major [M][F] (the reference returns its transpose rT [F][M]). */
int tfb_mlp8_fwd(const void* x8, const void* w8, const void* row, void* y, void* r, void* h8, long M, int d, int F,
                 void* stream);
/* tfb_mlp8_fwd with the block's residual add in the second GEMM's store: y = bf16(res + bf16(MLP(x))), res [M][d] bf16;
 * equal to tfb_mlp8_fwd followed by a bf16 add, bit for bit. Replaces the residual evacuation of _mlp8_fwd_nr_kernel
 * (round2/source/kernels/nki_mlp_nr8.py:1032: xo = bf16(x1 + y)). */
int tfb_mlp8_fwd_res(const void* x8, const void* w8, const void* row, const void* res, void* y, void* r, void* h8, long M,
                     int d, int F, void* stream);

/* Backward from dy8 = e5m2(dy s_dy) [M][d]: dx bf16 [M][d], dpre bf16 [M][F], h = bf16(r^2) [M][F] (NULL to skip),
 * dp8 [M][F] byte scratch. row = the backward row.
 * Replaces _mlp8_bwd_kernel / _mlp8_bwd_pc_kernel (nki_mlp_fused8.py:571, nki_mlp_l4t.py:496); op s2mlp8::bwd
 * (round2/source/train.py:6868), dw_mode "token" layout. */
int tfb_mlp8_bwd(const void* dy8, const void* r, const void* w8, const void* row, void* dx, void* h, void* dpre, void* dp8,
                 long M, int d, int F, void* stream);

/* out [O][D] (+)= (g8 [M][O]^T @ a8 [M][D]) * imm / (*s_g * *s_a): one weight gradient in fp8 from two token-major byte
 * tensors, contraction over the M tokens (fp32 accumulation over all of them, one rounding). (fmt_g, fmt_a) = (1, 0): an
 * e5m2 gradient against the forward's e4m3 activation bytes, or (0, 1). s_g, s_a: device fp32 scalars (the power-of-two
 * scales the bytes were cast at; NULL = 1). out bf16 (out_f32 = 0) or fp32, accumulate = 1 adds into it.
 * M, O, D multiples of 128; workspace >= splits * O * D * 4 bytes (256 MB always suffices).
 * Replaces dw8_grad (round2/source/train.py:8185; attn8_weight_grad 8232) = nki_dw8.py:323 emulate_dw / _dw8_kernel. */
int tfb_gemm_fp8_tn(const void* g8, int fmt_g, const void* a8, int fmt_a, const void* s_g, const void* s_a, float imm, void* out,
                    long M, int O, int D, int out_f32, int accumulate, void* workspace, long workspace_bytes, void* stream);

/* tfb_mlp8_bwd that also writes hq8 [M][F] = e4m3(min(bf16(r^2) * s_h, hq_limit)) (NULL to skip): the g-side operand of
 * the fp8 weight gradient of w_proj (format E4M3C of nki_dw8.py:312-320; round2/source/train.py:8226). dpre may be NULL
 * here: with both weight gradients in fp8 (tfb_mlp8_dw8) nothing reads the bf16 dpre, only its bytes dp8. */
int tfb_mlp8_bwd_q(const void* dy8, const void* r, const void* w8, const void* row, void* dx, void* h, void* dpre, void* dp8,
                   void* hq8, float hq_limit, long M, int d, int F, void* stream);

/* Both MLP weight gradients in fp8 from byte tensors the forward and backward already hold (token-major [M][.]):
 * dw_fc [F][d] = ((dp8^T @ x8) / (s_dp * x_scale)), dp8 = e5m2(dpre s_dp) from tfb_mlp8_bwd, x8 = e4m3(x x_scale);
 * dw_proj [d][F] = ((dy8^T @ hq8) / (s_dy * s_h)), dy8 = e5m2(dy s_dy), hq8 from tfb_mlp8_bwd_q. row = the backward row.
 * Outputs bf16 (out_f32 = 0) or fp32, optionally accumulated into (one rounding); fp32 accumulation over all tokens;
 * workspace >= splits * d * F * 4 bytes (256 MB always suffices). Shapes as tfb_mlp8_fwd. x_scale_dev (not NULL): the
 * activation scale as a device fp32 scalar instead of x_scale, as in tfb_mlp8_forward_scales.
 * Replaces mlp8_weight_grads under the fp8 weight-gradient switch (round2/source/train.py:8209-8229: dw8_grad twice,
 * nki_dw8.py:323 emulate_dw / _dw8_kernel) and R1's fp8 dW rows (round1/source/train.py:3182 run_tn_fp8). */
int tfb_mlp8_dw8(const void* x8, const void* dp8, const void* hq8, const void* dy8, const void* row, float x_scale, void* dw_fc,
                 void* dw_proj, long M, int d, int F, int out_f32, int accumulate, void* workspace, long workspace_bytes,
                 const void* x_scale_dev, void* stream);

/* ---- fp8 projections (attention QKV / output projection in fp8) -----------------------------------------------------
 * out8 [R][C], outT8 [C][R] = e4m3(w [R][C] * *scale_ptr): a weight pre-cast once per optimizer step in both byte layouts.
 * Replaces precast_ref (round2/source/kernels/nki_attn_tt8g.py:795). */
int tfb_precast8(const void* w, const void* scale_ptr, void* out8, void* outT8, int R, int C, void* stream);
/* out [M][N] bf16 = bf16((a8 [M][K] @ b8 [N][K]^T) * dq), a8 e4m3 (fmt_a 0) or e5m2 (fmt_a 1), b8 e4m3;
 * dq = dq_imm * *dq_a * *dq_b (device fp32 scalars or NULL). M, N, K % 128 == 0.
 * Replaces _proj8_fwd_kernel / _proj8_bwd_kernel (emulate_fwd, emulate_bwd: nki_attn_tt8g.py:745-757). */
int tfb_gemm_fp8(const void* a8, int fmt_a, const void* b8, const void* dq_a, const void* dq_b, float dq_imm, void* out,
                 long M, int N, int K, void* stream);
/* tfb_gemm_fp8 (e4m3 activations) with the residual add in the store: out = bf16(res + bf16((a8 @ b8^T) * dq)).
 * Replaces _proj8_fwd_ra_kernel (round2/source/kernels/nki_attn_nr8.py:1003). */
int tfb_gemm_fp8_res(const void* a8, const void* b8, const void* dq_a, const void* dq_b, float dq_imm, const void* res,
                     void* out, long M, int N, int K, void* stream);

/* dw [d][F] (+)= dy^T @ bf16(r^2) (bf16 GEMM over the tokens, h never materialised). workspace fp32 split-K scratch.
 * Replaces the dw_proj half of weight_grads (nki_mlp_fused8.py:706-711) / l4_weight_grads (nki_mlp_l4t.py:932). */
int tfb_mlp_dw_proj(const void* dy, const void* r, void* dw, long M, int d, int F, int out_f32, int accumulate,
                    void* workspace, long workspace_bytes, void* stream);

/* qkv [M][N] = rope(x [M][K] @ w [N][K]^T): the fused attention projection with the rotary embedding (half-split,
 * heads of 64) of its first rot_cols columns applied in the GEMM epilogue; row m is token m % T; cos_t, sin_t bf16
 * [T][32]. Equals tfb_gemm_bf16 followed by tfb_rope bit for bit. Replaces the c_attn projection + the rotation inside
 * nki_rope_attention (round1/source/train.py:8197, 4188-4193) as one launch. */
int tfb_qkv_rope_fwd(const void* x, const void* w, const void* cos_t, const void* sin_t, void* out, int M, int N, int K, int T,
                     int rot_cols, void* stream);

/* ---- attention ----------------------------------------------------------------------------------------------------
 * Causal flash attention, bf16. Every tensor comes with host long[3] element strides (batch, head, token); head dim
 * contiguous; so q/k/v can be [B,H,T,D], [B,T,H,D] or thirds of a fused [B,T,3C] projection. lse fp32 [B*H][T].
 * T % 128 == 0, D == 64 or 128.
 * Replaces _attn_fwd_kernel behind nki_causal_attention (round1/source/train.py:7536, 8069;
 * round2/source/kernels/nki_attn_bandpro.py:1850); op s2attn::*_fwd (round2/source/train.py:4988). */
int tfb_attn_fwd(const void* q, const long* q_strides, const void* k, const long* k_strides, const void* v,
                 const long* v_strides, void* o, const long* o_strides, void* lse, int B, int H, int T, int D, float scale,
                 void* stream);

/* dq, dk, dv from (q, k, v, o, do, lse); delta fp32 [2][B*H][T] scratch (the rows' -sum(dO O) and -lse / scale, which the
 * first kernel, dQ, leaves for the second).
 * Replaces _attn_bwd_kernel / NkiAttnFn.backward (round1/source/train.py:7591, 8036). */
int tfb_attn_bwd(const void* q, const long* q_strides, const void* k, const long* k_strides, const void* v,
                 const long* v_strides, const void* o, const long* o_strides, const void* d_o, const long* do_strides,
                 void* dq, const long* dq_strides, void* dk, const long* dk_strides, void* dv, const long* dv_strides,
                 const void* lse, void* delta, int B, int H, int T, int D, float scale, void* stream);
/* tfb_attn_bwd for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): the same kernels and results, with the delta scratch taken from a static device
 * array inside the library (8 MiB per GPU, held until the process ends) instead of from the caller. It allocates and
 * frees nothing. B * H * T <= tfb_attn_bwd_static_max_rows() (1,048,576), otherwise status 4 and the caller uses
 * tfb_attn_bwd. All calls on one GPU share that GPU's array: calls that overlap on one GPU (two streams) race.
 * The first call on a device looks up the array's address (hipGetSymbolAddress): make one call eagerly on each device
 * before capturing a call into a HIP graph.
 * Has no counterpart in the reference (its kernels allocate their own outputs and scratch through the NKI runtime). */
long tfb_attn_bwd_static_max_rows(void);
int tfb_attn_bwd_static(const void* q, const long* q_strides, const void* k, const long* k_strides, const void* v,
                        const long* v_strides, const void* o, const long* o_strides, const void* d_o, const long* do_strides,
                        void* dq, const long* dq_strides, void* dk, const long* dk_strides, void* dv, const long* dv_strides,
                        const void* lse, int B, int H, int T, int D, float scale, void* stream);
/* The same, with the inverse RoPE rotation (cos_t, sin_t bf16 [T][D/2]) applied to dq and dk on their way out: the
 * backward half of attention over a rotated fused projection. D == 64; TFB_ERR_SHAPE otherwise (caller runs tfb_rope).
 * Replaces NkiRopeAttnFn.backward / s2attn::rope_attn_bwd (round1/source/train.py:8135; round2/source/train.py:5040). */
int tfb_attn_bwd_rope(const void* q, const long* q_strides, const void* k, const long* k_strides, const void* v,
                      const long* v_strides, const void* o, const long* o_strides, const void* d_o, const long* do_strides,
                      void* dq, const long* dq_strides, void* dk, const long* dk_strides, void* dv, const long* dv_strides,
                      const void* lse, void* delta, const void* cos_t, const void* sin_t, int B, int H, int T, int D,
                      float scale, void* stream);
/* The tile band of the reference's windowed layers (band_mask, round2/source/kernels/nki_attn_bandpro.py:1654-1658;
 * kernels _attn_rope_fwd_kernel_band / _attn_rope_bwd_kernel_band, ops s2attn::rope_attn_fwd_band / _bwd_band
 * round2/source/train.py:4925, 5040-5068): with nw > 0 a query of 128-token tile i sees the keys k <= q of tiles
 * i - nw + 1 .. i only (the key loops start later / end earlier; the diagonal tile stays causally masked); nw = 0 is
 * tfb_attn_fwd / tfb_attn_bwd_rope. Other arguments as there. */
int tfb_attn_fwd_band(const void* q, const long* q_strides, const void* k, const long* k_strides, const void* v,
                      const long* v_strides, void* o, const long* o_strides, void* lse, int B, int H, int T, int D, float scale,
                      int nw, void* stream);
int tfb_attn_bwd_band(const void* q, const long* q_strides, const void* k, const long* k_strides, const void* v,
                      const long* v_strides, const void* o, const long* o_strides, const void* go, const long* go_strides,
                      void* dq, const long* dq_strides, void* dk, const long* dk_strides, void* dv, const long* dv_strides,
                      const void* lse, void* delta, const void* cos_t, const void* sin_t, int B, int H, int T, int D, float scale,
                      int nw, void* stream);

/* ---- loss head ------------------------------------------------------------------------------------------------------
 * loss[row] = row_w[row] * (lse - s_target), lse[row] = log sum exp(s), s = softcap tanh(x / softcap) (softcap <= 0:
 * s = x); a target outside [0, V) (the reference's ignore_index -1, or any id beyond the vocabulary) = ignored row:
 * loss 0, gradient 0, never an address. logits bf16 [rows][V]; targets int64 (idx64) or int32.
 * Replaces _loss_fwd_kernel behind fused_loss (round1/source/train.py:4543, 4691) and _lh_fwd_kernel
 * (round2/source/train.py:5238; host chunked_loss_mean 6364). */
int tfb_loss_fwd(const void* logits, const void* targets, int idx64, const void* row_w, void* loss, void* lse, long rows,
                 int V, float softcap, void* stream);

/* dlogits = grow[row] (softmax - onehot) (1 - tanh^2), bf16; may alias logits.
 * Replaces _loss_bwd_kernel (round1/source/train.py:4584) / _lh_bwd_kernel (round2/source/train.py:5297). */
int tfb_loss_bwd(const void* logits, const void* targets, int idx64, const void* lse, const void* grow, void* dlogits,
                 long rows, int V, float softcap, void* stream);

/* Several targets per row and / or label smoothing: targets [K][rows] (int64 or int32; < 0 = weight 0), row_w fp32
 * [K][rows], 1 <= K <= 8, 0 <= eps < 1:  loss[row] = sum_k row_w[k][row] (lse - (1 - eps) s_{t_k} - (eps / V) sum_v s_v).
 * K > 1, eps = 0 replaces _loss_multi_fwd_kernel behind fused_loss_multi(logits, tg, rw, softcap)
 * (round1/source/train.py:4725, 4908); K = 1, eps > 0 replaces _lh_fwd_ls_kernel (round2/source/train.py:5697; host
 * chunked_loss_mean(smooth=True) 6364, the mean and per-token weights being row weights). */
int tfb_loss_multi_fwd(const void* logits, const void* targets, int idx64, const void* row_w, int K, float eps, void* loss,
                       void* lse, long rows, int V, float softcap, void* stream);

/* dlogits = g[row] (1 - tanh^2) (W softmax - (1 - eps) sum_k row_w[k][row] [v = t_k] - W eps / V), W = sum_k row_w[k][row];
 * bf16, may alias logits. Replaces _loss_multi_bwd_kernel (round1/source/train.py:4778) and _lh_bwd_ls_kernel
 * (round2/source/train.py:5767). */
int tfb_loss_multi_bwd(const void* logits, const void* targets, int idx64, const void* row_w, int K, float eps, const void* lse,
                       const void* g, void* dlogits, long rows, int V, float softcap, void* stream);

/* w fp32 [rows] = each row's weight in the reduced loss: valid / max(1, #valid) when mean != 0 (the mean over the rows
 * whose target counts), valid otherwise; valid = 0 <= t < V, the rows the loss kernels give a loss to (V <= 0: no upper
 * bound). One launch for the compare / sum / clamp / divide the caller of fused_loss(reduction=) makes on the host side
 * (round1/source/train.py:4703-4707 scales the row losses there). */
int tfb_loss_row_weights(const void* targets, int idx64, void* w, long rows, int mean, int V, void* stream);

/* tfb_loss_fwd followed by tfb_loss_bwd with grow = row_w (an upstream gradient of one), in place and in ONE pass over the
 * logits (a row is held in a workgroup's registers, V <= 65536; TFB_ERR_SHAPE beyond): loss and lse as tfb_loss_fwd writes
 * them, logits overwritten by d logits = row_w (softmax - onehot) (1 - tanh^2), all three bit-equal to the two calls.
 * Replaces _loss_fwd_kernel + _loss_bwd_kernel (round1/source/train.py:4543, 4584) when the loss is differentiated. */
int tfb_loss_fwd_bwd(void* logits, const void* targets, int idx64, const void* row_w, void* loss, void* lse, long rows, int V,
                     float softcap, void* stream);

/* logits = x @ W^T (x [rows][d], W [V][d]) with the row log-sum-exp reduced in the GEMM epilogue, then loss / lse as
 * tfb_loss_fwd. part: fp32 scratch of rows * (V / 64) * 2 elements. rows, V multiples of 128, d of 64.
 * Replaces the lm_head matmul + loss forward pair (round1/source/train.py:8668, 9191-9212). */
int tfb_lmhead_fwd(const void* x, const void* W, const void* targets, int idx64, const void* row_w, void* logits, void* part,
                   void* loss, void* lse, long rows, int d, int V, float softcap, void* stream);

/* ---- mixture of experts (top-1 / top-2, all experts on this GPU, dropless ragged slots) -------------------------------
 * Slot buffer: expert e's assignments are contiguous rows, in token order, padded to a multiple of 128 (zero rows).
 * Tables (device int32): cnt[E], seg[E+1] padded segment offsets, tile_expert[rmax/128] (-1 beyond the extent),
 * slot[N][topk], tok[rmax] (-1 = padding), ksel[rmax]. rmax = tfb_moe_max_rows(N, E, topk) (host helper). */
long tfb_moe_max_rows(long N, int E, int topk);

/* p = softmax(h Wr^T + bias) fp32 [N][E] (logits optional), the top-k experts by first maximum (ties low) and gates
 * (renormalised over the two at k = 2, the probability at k = 1). h bf16 [N][d], wr fp32 [E][d]; E <= 16.
 * Replaces the router matmul + moe_route / moe_tournament (round2/source/train.py:10505-10553, 10961). */
int tfb_moe_route(const void* h, const void* wr, const void* bias, void* logits, void* p, void* idx, void* gate, long N, int d,
                  int E, int topk, void* stream);

/* The slot tables from idx. scratch: int32 [ceil(N/64) * E].
 * Replaces moe_positions + moe_gather_tables (round2/source/train.py:10555-10634) without a capacity (nothing is dropped). */
int tfb_moe_tables(const void* idx, void* cnt, void* seg, void* tile_expert, void* slot, void* tok, void* ksel, void* scratch,
                   long N, int E, int topk, long rmax, void* stream);

/* The slot tables under the reference's per-sequence capacity: the N tokens are N / T sequences of T; of one sequence's
 * assignments to one expert (both choices, token order) the first cap keep a row, the rest get slot -1 (they read the
 * reference's zero row and receive no gradient). cnt [E]: kept assignments; cnt_all [E]: all of them (the load-balance
 * term's shares). scratch: int32 [2 * ceil(N/64) * E]. Status 1 unless T % 64 == 0, N % T == 0, cap >= 1.
 * Replaces moe_positions + moe_gather_tables with their capacity (round2/source/train.py:10555-10634: pos < cap keeps). */
int tfb_moe_tables_cap(const void* idx, void* cnt, void* cnt_all, void* seg, void* tile_expert, void* slot, void* tok, void* ksel,
                       void* scratch, long N, long T, int cap, int E, int topk, long rmax, void* stream);

/* xs bf16 [rmax][d] = h[tok] (zero padding rows) and xs8 = e4m3(xs * scale) (scale_ptr device fp32 or scale_imm; either
 * output may be NULL: bf16 experts take no fp8 copy, fp8 experts with fp8 weight gradients no bf16 one).
 * Replaces MoeDispatch2.forward (round2/source/train.py:10652-10660). */
int tfb_moe_gather(const void* h, const void* tok, const void* scale_ptr, float scale_imm, void* xs, void* xs8, long rmax, int d,
                   void* stream);

/* Grouped fp8 expert MLP: x8 [rmax][d] -> y bf16 [rmax][d], r bf16 [rmax][F]; w8 uint8 [E][4][F*d] (tfb_mlp8_precast per
 * expert), rows fp32 [E][16]; h8 [rmax][F] byte scratch.
 * Replaces moe_experts8_local / moe_expert8_mlp (round2/source/train.py:10731-10776). */
int tfb_moe_mlp8_fwd(const void* x8, const void* w8, const void* rows, const void* tile_expert, void* y, void* r, void* h8,
                     long rmax, int d, int F, void* stream);
int tfb_moe_mlp8_bwd(const void* dy8, const void* r, const void* w8, const void* rows, const void* tile_expert, void* dx,
                     void* dpre, void* dp8, long rmax, int d, int F, void* stream);
/* tfb_moe_mlp8_bwd for the fp8 weight gradients: dpre may be NULL (they read dp8), and with hq8 non-NULL also
 * hq8 [rmax][F] = e4m3(min(bf16(r^2) s_h, hq_limit)) at each expert's own s_h (tfb_mlp8_bwd_q, grouped). */
int tfb_moe_mlp8_bwd_q(const void* dy8, const void* r, const void* w8, const void* rows, const void* tile_expert, void* dx,
                       void* dpre, void* dp8, void* hq8, float hq_limit, long rmax, int d, int F, void* stream);
/* The experts' two weight gradients in fp8 over each expert's row segment [seg[e], seg[e+1]) of the grouped byte buffers:
 * dw_fc [E][F][d] (+)= bf16((dp8_e^T @ xs8_e) / (s_dp[e] x_scale)), dw_proj [E][d][F] (+)= bf16((dy8_e^T @ hq8_e) /
 * (s_dy[e] s_h[e])); rows fp32 [E][16] = the backward call's rows; bf16 or fp32 outputs, optionally accumulated into.
 * Replaces mlp8_weight_grads under its fp8 weight-gradient switch (round2/source/train.py:8209-8229) inside the experts'
 * backward (moe_expert8_mlp, round2/source/train.py:10731), expert by expert. */
int tfb_moe_dw8(const void* xs8, const void* dp8, const void* hq8, const void* dy8, const void* rows, float x_scale,
                const void* seg, void* dw_fc, void* dw_proj, int E, int d, int F, int out_f32, int accumulate, void* stream);

/* dw_fc [E][F][d] (+)= dpre_e^T xs_e, dw_proj [E][d][F] (+)= dys_e^T bf16(r_e^2) over each expert's row segment.
 * Replaces the per-expert weight_grads (round2/source/kernels/nki_mlp_fused8.py:706-711). */
int tfb_moe_dw(const void* dpre, const void* xs, const void* dys, const void* r, const void* seg, void* dw_fc, void* dw_proj,
               int E, int d, int F, int out_f32, int accumulate, void* stream);
/* The routed experts in bf16 (every expert on this GPU) on the grouped buffers: each expert applies
 * F.linear(relu(F.linear(x, w_fc[e])).square(), w_proj[e]) to its rows with the bf16 roundings of those four operations.
 * xs bf16 [rmax][d], w_fc bf16 [E][F][d], w_proj bf16 [E][d][F], tile_expert int32 [rmax/128] -> ys bf16 [rmax][d],
 * r bf16 [rmax][F] = relu(pre), h bf16 [rmax][F] = r^2 (both kept for the backward). d, F multiples of 128.
 * Replaces moe_experts_local / the kit's expression of moe_expert_mlp (round2/source/train.py:10716-10727, 10711). */
int tfb_moe_mlp_fwd(const void* xs, const void* w_fc, const void* w_proj, const void* tile_expert, void* ys, void* r, void* h,
                    long rmax, int d, int F, void* stream);
/* Its backward: dpre bf16 [rmax][F] = bf16(bf16(dys w_proj[e]) 2 r), dxs bf16 [rmax][d] = dpre w_fc[e] (autograd through the
 * same expression); the weight gradients are tfb_moe_dw(dpre, xs, dys, r, ...). */
int tfb_moe_mlp_bwd(const void* dys, const void* r, const void* w_fc, const void* w_proj, const void* tile_expert, void* dxs,
                    void* dpre, long rmax, int d, int F, void* stream);

/* out bf16 [N][d] = sum_k bf16(gate_k) ys[slot_k] (the eager bf16 expression's roundings).
 * Replaces MoeCombine2.forward + the gated sum (round2/source/train.py:10672-10676, 10990-10992). */
int tfb_moe_combine(const void* ys, const void* slot, const void* gate, void* out, long N, int d, int topk, void* stream);

/* dys bf16 [rmax][d] = bf16(gate_k) dout[tok]; dgate fp32 [N][topk] = sum_d dout ys.
 * Replaces MoeCombine2.backward (round2/source/train.py:10678-10688). */
int tfb_moe_combine_bwd(const void* dout, const void* ys, const void* tok, const void* ksel, const void* gate, void* dys,
                        void* dgate, long rmax, int d, int topk, void* stream);

/* tfb_moe_combine_bwd that also leaves rowmax fp32 [rmax] = max |dys[row]| of the rounded values (0 for a padding row), so
 * that the experts' backward scales (tfb_moe_backward_scales_rowmax) need no pass of their own over dys.
 * Replaces MoeCombine2.backward (round2/source/train.py:10678-10688) + the amax(dy) of backward_scales
 * (round2/source/kernels/nki_mlp_fused8.py:803). */
int tfb_moe_combine_bwd_rowmax(const void* dout, const void* ys, const void* tok, const void* ksel, const void* gate, void* dys,
                               void* dgate, void* rowmax, long rmax, int d, int topk, void* stream);

/* dlogits fp32 [N][E] from dgate through the renormalisation and the softmax; dh bf16 [N][d] = dxs[slot_1] + dxs[slot_2] +
 * dlogits Wr; dwr fp32 [E][d] (+)= dlogits^T h, summed over 64 token chunks in a fixed order through scratch fp32 [64][E][d].
 * Replaces MoeDispatch2.backward (round2/source/train.py:10662-10666) and autograd through moe_route / the router matmul. */
int tfb_moe_route_bwd(const void* dgate, const void* p, const void* idx, const void* dxs, const void* slot, const void* h,
                      const void* wr, void* dlogits, void* dh, void* dwr, int dwr_accumulate, void* scratch, long N, int d, int E,
                      int topk, void* stream);
/* tfb_moe_route_bwd with the gradient of the auxiliary router terms folded into dlogits: the weighted sum
 * alpha lb + beta z of tfb_moe_aux_fwd received the gradient *gaux (device fp32 scalar); terms, lse as that call left them. */
int tfb_moe_route_bwd_aux(const void* dgate, const void* p, const void* idx, const void* dxs, const void* slot, const void* h,
                          const void* wr, void* dlogits, void* dh, void* dwr, int dwr_accumulate, void* scratch,
                          const void* terms, const void* lse, const void* gaux, float alpha, float beta, long N, int d, int E,
                          int topk, void* stream);
/* The router's auxiliary loss terms: terms fp32 [2 + E] = (lb = E sum_e f_e P_e, z = mean_n logsumexp(logits_n)^2, f_e),
 * f_e = cnt_e / (N topk) the share of the assignments that chose e (cnt: the slot tables' counts; no gradient), P_e the
 * mean router probability; lse fp32 [N] is kept for the backward; scratch fp32 [64 * 17].
 * Replaces moe_aux_terms (round2/source/train.py:10779-10788); its per-sequence term (R2_MOE_AUX_SEQ, 10789-10792) is
 * tfb_moe_aux_seq_fwd. */
int tfb_moe_aux_fwd(const void* p, const void* logits, const void* cnt, void* terms, void* lse, void* scratch, long N, int E,
                    int topk, void* stream);
/* The per-sequence balance term of moe_aux_terms (round2/source/train.py:10789-10792): term fp32 [1] = the mean over the
 * N / T sequences of E sum_e fs[b][e] ps[b][e]; fs fp32 [N / T][E] = each sequence's share of its T topk assignments per
 * expert (from idx int32 [N][topk], every selection counted whether a capacity later drops its row; no gradient; kept for
 * the backward), ps the sequence's mean router probability. scratch fp32 [N / T]. N % T == 0. */
int tfb_moe_aux_seq_fwd(const void* p, const void* idx, void* fs, void* term, void* scratch, long N, long T, int E, int topk,
                        void* stream);
/* tfb_moe_route_bwd_aux with that term as well: the weighted sum alpha lb + beta z + gamma seq received the gradient *gaux;
 * fs as tfb_moe_aux_seq_fwd left it. */
int tfb_moe_route_bwd_aux_seq(const void* dgate, const void* p, const void* idx, const void* dxs, const void* slot,
                              const void* h, const void* wr, void* dlogits, void* dh, void* dwr, int dwr_accumulate,
                              void* scratch, const void* terms, const void* lse, const void* gaux, float alpha, float beta,
                              const void* fs, float gamma, long T, long N, int d, int E, int topk, void* stream);

/* rows_out fp32 [E][16] = rows_in with the backward columns filled from each expert's amax over its rows of dys
 * (backward_scales per expert, round2/source/kernels/nki_mlp_fused8.py:803-813). amax_scratch: uint32 [E]. */
int tfb_moe_backward_scales(const void* dys, const void* tile_expert, const void* rows_in, void* rows_out, void* amax_scratch,
                            long rmax, int d, int E, void* stream);

/* The same rows from rowmax fp32 [rmax] (tfb_moe_combine_bwd_rowmax) and seg int32 [E + 1] (tfb_moe_tables): expert e's amax
 * is the maximum over rows seg[e] .. seg[e + 1]; bit-equal to tfb_moe_backward_scales on the same dys; d as there.
 * Replaces backward_scales per expert (round2/source/kernels/nki_mlp_fused8.py:803-813). */
int tfb_moe_backward_scales_rowmax(const void* rowmax, const void* seg, const void* rows_in, void* rows_out, int d, int E,
                                   void* stream);

/* out8 = fp8(x * rows[expert of the row's tile][col]); fmt 0 e4m3, 1 e5m2; padding tiles give zero bytes. */
int tfb_moe_quant(const void* x, const void* tile_expert, const void* rows, int col, int fmt, void* out8, long rmax, int d,
                  void* stream);

/* ---- Muon: Newton-Schulz ("Polar Express") orthogonalisation of a stack of gradient matrices -------------------------
 * Per matrix, held tall X [M][N] (M >= N): X0 = bf16(bf16(g) / d), then five times G = bf16(X^T X),
 * B = bf16(c G G + b G), X = bf16(X B + a X) with the (a, b, c) of `coeffs` (15 host floats), fp32 accumulation;
 * y = X5 in g's layout, v [K][M] = the sums of X5^2 along the N-long side (the NorMuon row statistic times N).
 * g fp32 [K][M][N] (wide 0) or [K][N][M] (wide 1: handled as the transposes); inv_d fp32 [K] device (1 / d). M, N % 128.
 * workspace: tfb_ns5_workspace_bytes(K, M, N) bytes of device memory. The whole stack takes 3 grouped GEMM launches per
 * iteration. Replaces _nsk_kernel(ga, gb, sc) -> ya, yb, va, vb (round2/source/kernels/nki_nsk.py:370; arithmetic
 * emulate_nsk :452) = the loop of muon_math_body (reference_ns :471); one call per stack. */
long tfb_ns5_workspace_bytes(int K, int M, int N);
int tfb_ns5(const void* g, const void* inv_d, const float* coeffs, void* y, void* v, int K, int M, int N, int wide,
            void* workspace, long workspace_bytes, void* stream);

/* ---- dense bf16 fused MLP ---------------------------------------------------------------------------------------------
 * x bf16 [M][d], w_fc bf16 [F][d], w_proj bf16 [d][F] (nn.Linear layouts) -> y bf16 [M][d] = bf16(h @ w_proj^T) with
 * r = bf16(relu(x @ w_fc^T)) (bf16 [M][F], token-major, saved for the backward) and h = bf16(r r) (bf16 [M][F], the second
 * GEMM's operand). M, d, F multiples of 128.
 * Replaces _mlp_fwd_kernel(x2, w_fc, w_proj, tb) -> (y, rT) (round2/source/kernels/nki_mlp_fused.py:242; arithmetic
 * emulate_forward :372); the reference saves r's transpose. */
int tfb_mlp_fwd(const void* x, const void* w_fc, const void* w_proj, void* y, void* r, void* h, long M, int d, int F,
                void* stream);
/* dy bf16 [M][d], r as the forward left it -> dx bf16 [M][d], dpre bf16 [M][F] = bf16(((dy @ w_proj) 2) r) (one rounding),
 * h bf16 [M][F] = bf16(r r) (optional, may be NULL): dpre and h are what the weight gradients contract (dpre^T x, dy^T h).
 * Replaces _mlp_bwd_kernel(dy2, rT, w_fc, w_proj, tb, dw_mode) -> (dx, h, dpre) with dw_mode 0
 * (round2/source/kernels/nki_mlp_fused.py:290; arithmetic emulate_backward :382, weight_grads :394). */
int tfb_mlp_bwd(const void* dy, const void* r, const void* w_fc, const void* w_proj, void* dx, void* h, void* dpre, long M,
                int d, int F, void* stream);

/* ---- gradient norm ---------------------------------------------------------------------------------------------------
 * out fp32 [4] = (sum of squares of g_bf16 [n_bf16], of g_f32 [n_f32], sqrt of their sum, min(clip / (norm + 1e-6), 1) or 1
 * when clip <= 0), left on the device; either buffer may be absent (NULL, 0). scratch: fp32
 * [tfb_gradnorm_scratch_floats()]. Two launches, sums in a fixed order.
 * Replaces _gradnorm_kernel (round1/source/train.py:1480) and the norm / clip-factor arithmetic of reduce_fused (:1634). */
long tfb_gradnorm_scratch_floats(void);
int tfb_gradnorm(const void* g_bf16, long n_bf16, const void* g_f32, long n_f32, float clip, void* scratch, void* out,
                 void* stream);

/* ---- mixer tail ------------------------------------------------------------------------------------------------------
 * x bf16 [nrows][C] (nrows = sequences of T tokens), lam a device fp32 scalar -> s1 = bf16(x + bf16(lam shift1(x))) where
 * shift1 hands token t the row of token t - 1 of its sequence (zeros at t = 0), xn2 = RMSNorm(s1) without weight, inv fp32
 * [nrows]. Replaces mix_tail's forward kernel _mix_fwd_kernel (round1/source/train.py:7097, wrapper :7308). */
int tfb_mix_tail_fwd(const void* x, const void* lam, void* s1, void* xn2, void* inv, long nrows, int C, int T, float eps,
                     void* stream);
/* gy (gradient of xn2), ge (gradient of s1), either may be NULL -> gx bf16 [nrows][C] = bf16(g[t] + bf16(lam g[t + 1])) with
 * g the tail norm's backward bf16(ge + inv (gy - s1 (gy . s1) inv^2 / C)) (g[t + 1] = 0 at a sequence's last token), and
 * dlam fp32 [1] = the fp32 sum of the bf16 products bf16(g shift1(x)). part: fp32 [tfb_norm_bwd_blocks(nrows)] scratch.
 * Replaces _mix_bwd_kernel (round1/source/train.py:7145). */
int tfb_mix_tail_bwd(const void* s1, const void* gy, const void* ge, const void* inv, const void* x, const void* lam, void* gx,
                     void* part, void* dlam, long nrows, int C, int T, void* stream);

#ifdef __cplusplus
}
#endif
#endif
