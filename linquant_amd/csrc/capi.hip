// ABI bookkeeping for liblinquant_hip.so.
#include <string.h>

#include "lq_common.h"
#include "../../include/linquant_hip.h"

extern "C" int lq_abi_version(void) { return 18; }

#define LQ_SIZE_OF(T) \
  if (strcmp(name, #T) == 0) return (int)sizeof(T)

extern "C" int lq_args_size(const char* name) {
  if (!name) return LQ_ERR_NULL;
  LQ_SIZE_OF(lq_chunk_cumsum_args);
  LQ_SIZE_OF(lq_chunk_state_value_args);
  LQ_SIZE_OF(lq_chunk_state_key_args);
  LQ_SIZE_OF(lq_state_passing_args);
  LQ_SIZE_OF(lq_bmm_chunk_args);
  LQ_SIZE_OF(lq_chunk_scan_args);
  LQ_SIZE_OF(lq_split_rotate_quant_xBC_args);
  LQ_SIZE_OF(lq_kron_hadamard_args);
  LQ_SIZE_OF(lq_fp16_to_int8_args);
  LQ_SIZE_OF(lq_causal_conv1d_args);
  LQ_SIZE_OF(lq_rmsnorm_gated_args);
  LQ_SIZE_OF(lq_absmax_args);
  LQ_SIZE_OF(lq_absmax_chunk_state_args);
  LQ_SIZE_OF(lq_absmax_cb_args);
  LQ_SIZE_OF(lq_qhad_transform_args);
  LQ_SIZE_OF(lq_rmsnorm_gated_qhad_args);
  LQ_SIZE_OF(lq_zoo_cumsum_args);
  LQ_SIZE_OF(lq_zoo_write_codes_args);
  LQ_SIZE_OF(lq_zoo_state_args);
  LQ_SIZE_OF(lq_zoo_output_args);
  LQ_SIZE_OF(lq_zoo_simple_gla_args);
  LQ_SIZE_OF(lq_zoo_chunk_forward_args);
  LQ_SIZE_OF(lq_zoo_gla_A_args);
  LQ_SIZE_OF(lq_zoo_wy_prep_args);
  LQ_SIZE_OF(lq_zoo_rotate_qkv_args);
  LQ_SIZE_OF(lq_zoo_rotate_quant_args);
  LQ_SIZE_OF(lq_ssd_combined_args);
  LQ_SIZE_OF(lq_probe_mfma_args);
  return LQ_ERR_SHAPE;
}
