/*
** The part of AnnI's backend ABI (num/gpu.h) that lies outside the optimizer
** step.  Exported so the library links wherever the reference's backends do;
** every entry gives the CPU stub's answer (num/gpu_stub.c), so the caller's own
** fallback runs.  See include/anni_gpu_unserved.h.
*/
#include "anni_gpu_unserved.h"

#define NOT_HERE	{ return -1; }
#define ANSWER(x)	{ return (x); }
#define NOTHING		{ }

static int g_sync_mode;

extern "C" {

void	gpu_set_sync_mode(int mode) { g_sync_mode = mode; }
int	gpu_sync_mode(void) ANSWER(g_sync_mode)
void	gpu_set_fp8(int) NOTHING
void	gpu_set_fp8_dgrad(int) NOTHING
int	gpu_fp8(void) ANSWER(0)

int	gpu_mat_mul(mat *, const mat *, const mat *) NOT_HERE
int	gpu_mat_mul_bias(mat *, const mat *, const mat *, const ann_real *) NOT_HERE
int	gpu_mat_mul_res(mat *, const mat *, const mat *, const ann_real *, const mat *) NOT_HERE
int	gpu_mat_mul_bias_relu(mat *, const mat *, const mat *, const ann_real *) NOT_HERE
void	gpu_grad_twins_clear(void) NOTHING
int	gpu_mat_mul_bt(mat *, const mat *, const mat *) NOT_HERE
int	gpu_mat_mul_bt_acc(mat *, const mat *, const mat *) NOT_HERE
int	gpu_mat_mul_bt_twin(mat *, const mat *, const mat *) NOT_HERE
int	gpu_mat_mul_at(mat *, const mat *, const mat *) NOT_HERE
int	gpu_mat_outer_add(mat *, const mat *, const mat *) NOT_HERE

int	gpu_layernorm_backward(mat *, const mat *, const ann_real *, const ann_real *,
		const ann_real *, int, int, ann_real *, ann_real *) NOT_HERE
int	gpu_layernorm_backward_acc(mat *, const mat *, const ann_real *, const ann_real *,
		const ann_real *, int, int, ann_real *, ann_real *) NOT_HERE
int	gpu_layernorm_backward_x(mat *, const mat *, const ann_real *, const ann_real *,
		const ann_real *, const ann_real *, int, int, ann_real *, ann_real *, int) NOT_HERE
int	gpu_layernorm_xhat(ann_real *, const ann_real *, const ann_real *, const ann_real *,
		int, int) NOT_HERE
int	gpu_layernorm_forward_ex(ann_real *, const ann_real *, const ann_real *,
		const ann_real *, ann_real *, ann_real *, ann_real *, int, int, double) NOT_HERE

int	gpu_ce_fetch_mean(double *, int) NOT_HERE
int	gpu_softmax_rows(ann_real *, int, int) NOT_HERE
int	gpu_softmax_bwd_rows(ann_real *, const ann_real *, const ann_real *, int, int) NOT_HERE
int	gpu_bias_row_add(ann_real *, const ann_real *, int, int) NOT_HERE
int	gpu_ce_delta_from_softmax(ann_real *, const int *, int, int, ann_real *, double *) NOT_HERE
int	gpu_ce_softmax_delta_bf16(ann_real *, const int *, int, int, const ann_real *,
		ann_real *, double *) NOT_HERE
int	gpu_ce_bias_fused(void) ANSWER(0)
int	gpu_ce_bf16_delta_done(const ann_real *) NOT_HERE
int	gpu_ce_nll_rows(const ann_real *, const int *, int, int, float *) NOT_HERE
int	gpu_posenc_add_packed(ann_real *, int, int, int) NOT_HERE
int	gpu_relu_backward(ann_real *, const ann_real *, int) NOT_HERE
int	gpu_ffn_relu_bwd_fused(mat *, const mat *, ann_real *) NOT_HERE
int	gpu_act_bf16_only(const mat *) ANSWER(0)
int	gpu_ffn_w1_finish(ann_real *, ann_real *, const ann_real *, int, int) NOT_HERE

int	gpu_attn_causal_fwd(mat *, mat *, const mat *, const mat *, const mat *, int, int, int,
		int) NOT_HERE
int	gpu_attn_flash_fwd(mat *, const mat *, const mat *, const mat *, int, int, int, int,
		mat *) NOT_HERE
int	gpu_attn_fa_fwd(mat *, const mat *, const mat *, const mat *, int, int, int, int,
		mat *) NOT_HERE
int	gpu_attn_fa_usable(int, int) ANSWER(0)
int	gpu_attn_fa_bwd(mat *, mat *, mat *, const mat *, const mat *, const mat *, const mat *,
		const mat *, const mat *, int, int, int, int) NOT_HERE
int	gpu_attn_qkv_bwd(mat *, mat *, mat *, mat *, const mat *, const mat *, const mat *,
		const mat *, const mat *) ANSWER(1)
int	gpu_attn_tiled_bwd(mat *, mat *, mat *, const mat *, const mat *, const mat *,
		const mat *, const mat *, const mat *, int, int, int, int) NOT_HERE
int	gpu_attn_causal_bwd(mat *, mat *, mat *, const mat *, const mat *, const mat *,
		const mat *, const mat *, int, int, int, int) NOT_HERE
int	gpu_attn_tc_fwd(mat *, mat *, const mat *, const mat *, const mat *, int, int, int,
		int) NOT_HERE
int	gpu_attn_tc_bwd(mat *, mat *, mat *, const mat *, mat *, const mat *, const mat *,
		const mat *, int, int, int, int) NOT_HERE
void	gpu_attn_qkv_bf16_hint(int, int) NOTHING
int	gpu_attn_qkv_fused(mat *, mat *, mat *, const mat *, const mat *, const mat *,
		const mat *) NOT_HERE
int	gpu_pack_seq_rows(ann_real *, const ann_real *, int, int, int) NOT_HERE
int	gpu_unpack_seq_rows(ann_real *, const ann_real *, int, int, int) NOT_HERE
void	gpu_attn_set_seqlens(const int *) NOTHING

int	gpu_mat_copy(mat *, const mat *) NOT_HERE
int	gpu_mat_add(mat *, const mat *) NOT_HERE
int	gpu_mat_add2(mat *, const mat *, const mat *) NOT_HERE
int	gpu_mat_axpy(mat *, double, const mat *) NOT_HERE
int	gpu_embed_lookup(mat *, const mat *, const int *, int, int, ann_real) NOT_HERE
int	gpu_embed_scatter(mat *, const mat *, const int *, int, int, ann_real) NOT_HERE

void	*gpu_copy_stream(void) ANSWER(nullptr)
int	gpu_graph_begin(void) NOT_HERE
int	gpu_graph_end(void) NOT_HERE
int	gpu_graph_replay(void) NOT_HERE
int	gpu_graph_replayable(void) ANSWER(0)
void	gpu_graph_destroy(void) NOTHING
void	gpu_graph_set_mode(int) NOTHING
int	gpu_graph_supported(void) ANSWER(0)
int	gpu_ids_stage(const int *, const int *, int) NOT_HERE
void	gpu_ids_unstage(void) NOTHING
const int	*gpu_ce_targets_staged(const int *, int, int) ANSWER(nullptr)

gpu_dec	*gpu_dec_create(int, int, int, int, int, int) ANSWER(nullptr)
int	gpu_dec_set_layer(gpu_dec *, int, const gpu_dec_layer_w *) NOT_HERE
int	gpu_dec_set_io(gpu_dec *, const ann_real *, const ann_real *, const ann_real *, int,
		ann_real) NOT_HERE
int	gpu_dec_kv_load(gpu_dec *, int, const ann_real *, const ann_real *, int) NOT_HERE
int	gpu_dec_step(gpu_dec *, int, int, ann_real *) NOT_HERE
void	gpu_dec_free(gpu_dec **g) { if (g) *g = nullptr; }

} /* extern "C" */
