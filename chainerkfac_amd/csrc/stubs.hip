// Entry points not implemented yet: they fail loudly.
#include "common.h"
#define NOT_YET(name) return kfac::fail(KFAC_EINVAL, name " is not implemented yet")
extern "C" size_t kfac_bn_workspace_bytes(int, int) { return 0; }
extern "C" int kfac_bn_grad_matrix_f32(const float *, const float *, int, int, int, float, float, int, int, float *, void *, size_t, void *) { NOT_YET("kfac_bn_grad_matrix_f32"); }
extern "C" int kfac_inverse_plan_create(int, const int32_t *, kfac_inverse_plan_t *) { NOT_YET("kfac_inverse_plan_create"); }
extern "C" size_t kfac_inverse_plan_workspace_bytes(kfac_inverse_plan_t) { return 0; }
extern "C" int kfac_inverse_plan_destroy(kfac_inverse_plan_t) { return 0; }
extern "C" int kfac_spd_inverse_batched_f32(kfac_inverse_plan_t, const float *const *, float *const *, int32_t *, void *, size_t, void *) { NOT_YET("kfac_spd_inverse_batched_f32"); }
extern "C" int kfac_damp_plan_create(int, const int32_t *, const int32_t *, kfac_damp_plan_t *) { NOT_YET("kfac_damp_plan_create"); }
extern "C" int kfac_damp_plan_destroy(kfac_damp_plan_t) { return 0; }
extern "C" int kfac_pi_damp_batched_f32(kfac_damp_plan_t, float *const *, float *const *, const double *, int, float *, void *) { NOT_YET("kfac_pi_damp_batched_f32"); }
extern "C" size_t kfac_precond_conn_workspace_bytes(int, int) { return 0; }
extern "C" int kfac_precond_conn_f32(const float *, int, const float *, int, const float *, const float *, float *, float *, void *, size_t, void *) { NOT_YET("kfac_precond_conn_f32"); }
extern "C" size_t kfac_precond_bn_workspace_bytes(int) { return 0; }
extern "C" int kfac_precond_bn_f32(const float *, int, const float *, int, const float *, int, float *, float *, int32_t *, void *, size_t, void *) { NOT_YET("kfac_precond_bn_f32"); }
