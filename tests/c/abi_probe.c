/*
** A C99 caller of the library, compiled with the reference's own flags (Makefile:21:
** -W -Wall -ansi -pedantic -std=c99): the four headers are plain C, the symbols link, and the
** host-only entry points answer.  Prints the learning rate at a few schedule steps, which the
** reference's test pins (tests/test_ann.c:866-879), and what the backend says about itself.
*/
#include <stdio.h>
#include "anni_gpu.h"
#include "anni_gpu_unserved.h"
#include "anni_adam.h"
#include "anni_bench.h"

int main(void)
{
	anni_tensor t[2];
	anni_adam_config cfg;
	anni_adam *opt;

	anni_lr_set_schedule(100, 1000, "cosine");
	anni_lr_set_sched_from(0);
	printf("lr %.17g %.17g %.17g %.17g\n", anni_lr_step(1.0, 0), anni_lr_step(1.0, 99),
	    anni_lr_step(1.0, 600), anni_lr_step(1.0, 1100));
	printf("backend %s available %d\n", gpu_backend_name(), gpu_available());
	t[0].n = 4096;
	t[0].flags = ANNI_T_DECAY | ANNI_T_TWIN;
	t[1].n = 64;
	t[1].flags = 0;
	cfg.grad_type = ANNI_F32;
	cfg.moment_type = ANNI_F32;
	cfg.twins = 1;
	cfg.skip_nonfinite = 1;
	cfg.grad_slots = 1;
	cfg.layout = ANNI_LAYOUT_AUTO;
	opt = anni_adam_create(t, 2, &cfg);
	if (!gpu_available()) {
		printf("create %s\n", opt ? "unexpected" : "declined");
		return opt ? 1 : 0;
	}
	if (!opt)
		return 1;
	opt->weight_decay = 0.1;
	opt->grad_clip = 1.0;
	if (anni_adam_step_scaled(opt, 1e-3, 1.0) != 0 || anni_adam_sync_stats(opt) != 0)
		return 1;
	printf("create ok n %ld t %d norm %g\n", (long)opt->n, opt->t, opt->last_grad_norm);
	anni_adam_free(&opt);
	return 0;
}
