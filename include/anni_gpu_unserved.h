/*
** anni_gpu_unserved.h -- the symbols of AnnI's backend ABI (num/gpu.h) that lie
** outside the optimizer step.  libanni_gpu_hip.so exports them so that it links
** wherever gpu_stub.o / gpu_cuda.o do, and each one answers what the
** reference's CPU stub answers (num/gpu_stub.c): int functions -1 ("use the CPU
** path"; the few predicates 0, gpu_attn_qkv_bwd 1 = "nothing pending"),
** pointer functions NULL, void functions nothing.  GEMM, attention, LayerNorm,
** softmax / cross-entropy, embedding, graph capture and decode are not this
** library's job.  Line numbers are those of num/gpu.h.
*/
#ifndef ANNI_GPU_UNSERVED_H__
#define ANNI_GPU_UNSERVED_H__

#include "anni_gpu.h"

#ifdef __cplusplus
extern "C" {
#endif

/* num/mat.h:10-16 -- only pointers to it cross this ABI. */
#ifndef MAT_H__
typedef struct mat {
	ann_real	*data;
	ann_real	*d_data;
	int		rows;
	int		cols;
	int		on_device;
} mat;
#endif

#ifndef GPU_SYNC_EAGER
#define GPU_SYNC_EAGER	0	/* :17-18 */
#define GPU_SYNC_BATCH	1
#endif

/* modes (:19-20, :30-32): remembered, otherwise without effect */
void	gpu_set_sync_mode(int mode);
int	gpu_sync_mode(void);
void	gpu_set_fp8(int on);
void	gpu_set_fp8_dgrad(int on);
int	gpu_fp8(void);

/* GEMM family (:81-100) */
int	gpu_mat_mul(mat *c, const mat *a, const mat *b);
int	gpu_mat_mul_bias(mat *c, const mat *a, const mat *b, const ann_real *bias);
int	gpu_mat_mul_res(mat *d, const mat *a, const mat *b, const ann_real *bias, const mat *res);
int	gpu_mat_mul_bias_relu(mat *c, const mat *a, const mat *b, const ann_real *bias);
void	gpu_grad_twins_clear(void);
int	gpu_mat_mul_bt(mat *c, const mat *a, const mat *b);
int	gpu_mat_mul_bt_acc(mat *c, const mat *a, const mat *b);
int	gpu_mat_mul_bt_twin(mat *c, const mat *a, const mat *b);
int	gpu_mat_mul_at(mat *c, const mat *a, const mat *b);
int	gpu_mat_outer_add(mat *dw, const mat *a, const mat *b);

/* LayerNorm (:102-119, :154-157) */
int	gpu_layernorm_backward(mat *dx, const mat *dy, const ann_real *gamma,
		const ann_real *x_hat, const ann_real *inv_std, int T, int d,
		ann_real *dgamma, ann_real *dbeta);
int	gpu_layernorm_backward_acc(mat *dx, const mat *dy, const ann_real *gamma,
		const ann_real *x_hat, const ann_real *inv_std, int T, int d,
		ann_real *dgamma, ann_real *dbeta);
int	gpu_layernorm_backward_x(mat *dx, const mat *dy, const ann_real *gamma,
		const ann_real *x, const ann_real *mean, const ann_real *inv_std,
		int T, int d, ann_real *dgamma, ann_real *dbeta, int accumulate);
int	gpu_layernorm_xhat(ann_real *x_hat, const ann_real *x, const ann_real *mean,
		const ann_real *inv_std, int T, int d);
int	gpu_layernorm_forward_ex(ann_real *y, const ann_real *x, const ann_real *gamma,
		const ann_real *beta, ann_real *x_hat, ann_real *mean, ann_real *inv_std,
		int T, int d, double eps);

/* softmax, cross-entropy, elementwise (:75, :142-148, :159-214) */
int	gpu_ce_fetch_mean(double *mean_ce, int rows);
int	gpu_softmax_rows(ann_real *rows, int n_rows, int n_cols);
int	gpu_softmax_bwd_rows(ann_real *dx, const ann_real *y, const ann_real *dy,
		int n_rows, int n_cols);
int	gpu_bias_row_add(ann_real *x, const ann_real *bias, int rows, int cols);
int	gpu_ce_delta_from_softmax(ann_real *probs, const int *tgt, int rows, int V,
		ann_real *db_host, double *mean_ce);
int	gpu_ce_softmax_delta_bf16(ann_real *logits, const int *tgt, int rows, int V,
		const ann_real *bias, ann_real *db_host, double *mean_ce);
int	gpu_ce_bias_fused(void);
int	gpu_ce_bf16_delta_done(const ann_real *logits);
int	gpu_ce_nll_rows(const ann_real *logits, const int *tgt, int rows, int V, float *out);
int	gpu_posenc_add_packed(ann_real *x, int B, int T, int D);
int	gpu_relu_backward(ann_real *dx, const ann_real *x_pre_relu_or_mask, int n);
int	gpu_ffn_relu_bwd_fused(mat *dh, const mat *hidden, ann_real *db1_host);
int	gpu_act_bf16_only(const mat *m);
int	gpu_ffn_w1_finish(ann_real *hidden, ann_real *pre, const ann_real *bias, int rows,
		int cols);

/* attention (:223-287) */
int	gpu_attn_causal_fwd(mat *concat, mat *w, const mat *q, const mat *k, const mat *v,
		int B, int T, int H, int dh);
int	gpu_attn_flash_fwd(mat *concat, const mat *q, const mat *k, const mat *v, int B,
		int T, int H, int dh, mat *lse);
int	gpu_attn_fa_fwd(mat *concat, const mat *q, const mat *k, const mat *v, int B, int T,
		int H, int dh, mat *lse);
int	gpu_attn_fa_usable(int T, int dh);
int	gpu_attn_fa_bwd(mat *dq, mat *dk, mat *dv, const mat *dconcat, const mat *concat,
		const mat *q, const mat *k, const mat *v, const mat *lse, int B, int T,
		int H, int dh);
int	gpu_attn_qkv_bwd(mat *dx, mat *dwq, mat *dwk, mat *dwv, const mat *x_in,
		const mat *dq, const mat *wq, const mat *wk, const mat *wv);
int	gpu_attn_tiled_bwd(mat *dq, mat *dk, mat *dv, const mat *dconcat, const mat *concat,
		const mat *q, const mat *k, const mat *v, const mat *lse, int B, int T,
		int H, int dh);
int	gpu_attn_causal_bwd(mat *dq, mat *dk, mat *dv, const mat *dconcat, const mat *w,
		const mat *q, const mat *k, const mat *v, int B, int T, int H, int dh);
int	gpu_attn_tc_fwd(mat *concat, mat *w, const mat *q, const mat *k, const mat *v,
		int B, int T, int H, int dh);
int	gpu_attn_tc_bwd(mat *dq, mat *dk, mat *dv, const mat *dconcat, mat *w, const mat *q,
		const mat *k, const mat *v, int B, int T, int H, int dh);
void	gpu_attn_qkv_bf16_hint(int T, int dh);
int	gpu_attn_qkv_fused(mat *q, mat *k, mat *v, const mat *x, const mat *wq,
		const mat *wk, const mat *wv);
int	gpu_pack_seq_rows(ann_real *dst, const ann_real *src, int B, int T, int D);
int	gpu_unpack_seq_rows(ann_real *dst, const ann_real *src, int B, int T, int D);
void	gpu_attn_set_seqlens(const int *seqlens);

/* residency helpers, embedding (:293-309) */
int	gpu_mat_copy(mat *dst, const mat *src);
int	gpu_mat_add(mat *dst, const mat *src);
int	gpu_mat_add2(mat *dst, const mat *a, const mat *b);
int	gpu_mat_axpy(mat *y, double a, const mat *x);
int	gpu_embed_lookup(mat *out, const mat *table, const int *ids, int n, int tied,
		ann_real scale);
int	gpu_embed_scatter(mat *dtable, const mat *dout, const int *ids, int n, int tied,
		ann_real scale);

/* copy stream, graph capture, staged ids (:316, :339-349) */
void	*gpu_copy_stream(void);
int	gpu_graph_begin(void);
int	gpu_graph_end(void);
int	gpu_graph_replay(void);
int	gpu_graph_replayable(void);
void	gpu_graph_destroy(void);
void	gpu_graph_set_mode(int on);
int	gpu_graph_supported(void);
int	gpu_ids_stage(const int *ids, const int *alias, int n);
void	gpu_ids_unstage(void);
const int	*gpu_ce_targets_staged(const int *ids, int B, int T);

/* single-stream decode (:358-387) */
#ifndef GPU_H__
typedef struct gpu_dec_layer_w {
	const ann_real	*wq, *wk, *wv, *wo, *w1, *w2;
	const ann_real	*ln1_g, *ln1_b, *ln2_g, *ln2_b, *b1, *b2;
	double		eps1, eps2;
} gpu_dec_layer_w;
typedef struct gpu_dec gpu_dec;
#endif
gpu_dec	*gpu_dec_create(int n_layers, int d_model, int d_ff, int vocab, int max_T,
		int n_heads);
int	gpu_dec_set_layer(gpu_dec *g, int i, const gpu_dec_layer_w *w);
int	gpu_dec_set_io(gpu_dec *g, const ann_real *embed_dev, const ann_real *w_head_dev,
		const ann_real *b_head_host, int tied, ann_real scale);
int	gpu_dec_kv_load(gpu_dec *g, int layer, const ann_real *k_host, const ann_real *v_host,
		int n);
int	gpu_dec_step(gpu_dec *g, int id, int pos, ann_real *logits);
void	gpu_dec_free(gpu_dec **g);

#ifdef __cplusplus
}
#endif
#endif
