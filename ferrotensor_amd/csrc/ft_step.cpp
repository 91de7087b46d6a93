#include "ft_common.h"
extern "C" {
int ft_model_create(ft_context*, const ft_model_config*, ft_model**) { return ft_set_error(FT_ERR_INVALID, "not implemented"); }
int ft_model_destroy(ft_model*) { return FT_OK; }
int ft_model_set_tensor(ft_model*, const char*, const float*, const size_t*, int) { return ft_set_error(FT_ERR_INVALID, "not implemented"); }
int ft_model_set_lora(ft_model*, const char*, const float*, const float*, size_t, float) { return ft_set_error(FT_ERR_INVALID, "not implemented"); }
int ft_model_param_count(ft_model*, size_t*) { return ft_set_error(FT_ERR_INVALID, "not implemented"); }
int ft_model_param_info(ft_model*, size_t, const char**, size_t*) { return ft_set_error(FT_ERR_INVALID, "not implemented"); }
int ft_model_read_param(ft_model*, size_t, float*) { return ft_set_error(FT_ERR_INVALID, "not implemented"); }
int ft_model_read_grad(ft_model*, size_t, float*) { return ft_set_error(FT_ERR_INVALID, "not implemented"); }
int ft_model_forward_logits(ft_model*, const uint32_t*, size_t, size_t, float*) { return ft_set_error(FT_ERR_INVALID, "not implemented"); }
int ft_trainer_create(ft_model*, const ft_trainer_config*, ft_trainer**) { return ft_set_error(FT_ERR_INVALID, "not implemented"); }
int ft_trainer_destroy(ft_trainer*) { return FT_OK; }
int ft_trainer_train_chunk(ft_trainer*, const uint32_t*, const uint32_t*, const uint8_t*, size_t, size_t, int, ft_step_stats*, float*) { return ft_set_error(FT_ERR_INVALID, "not implemented"); }
}
