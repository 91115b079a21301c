// Library-wide pieces of libfastcache_hip: ABI version, per-thread error text, view validation.
#include "fc_common.h"

static thread_local char g_err[512] = "";

void fc_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

extern "C" int fc_abi_version(void) { return FC_ABI_VERSION; }
extern "C" const char* fc_last_error(void) { return g_err; }

int fc_check_view(const fc_kv_view* v, const char* who) {
  FC_REQUIRE(v != nullptr, FC_EINVAL, "%s: null view", who);
  FC_REQUIRE(v->base != nullptr, FC_EINVAL, "%s: null base pointer", who);
  FC_REQUIRE(v->dtype == FC_F32 || v->dtype == FC_F16 || v->dtype == FC_BF16, FC_EINVAL,
             "%s: unknown dtype %d", who, v->dtype);
  FC_REQUIRE(v->head_dim == FC_HEAD_DIM, FC_EUNSUPPORTED, "%s: head_dim %d (only %d is built)", who,
             v->head_dim, FC_HEAD_DIM);
  FC_REQUIRE(v->num_layers > 0 && v->batch > 0 && v->num_kv_heads > 0, FC_EINVAL,
             "%s: layers/batch/heads must be positive (%d, %d, %d)", who, v->num_layers, v->batch,
             v->num_kv_heads);
  FC_REQUIRE(v->max_seq_len >= 0, FC_EINVAL, "%s: negative max_seq_len", who);
  FC_REQUIRE(v->batch <= 65535 && v->num_layers <= 65535, FC_EUNSUPPORTED,
             "%s: batch/layers beyond grid limits", who);
  if (v->block_tables) {
    FC_REQUIRE(v->block_size > 0, FC_EINVAL, "%s: block_size must be positive", who);
    FC_REQUIRE((int64_t)v->table_stride * v->block_size >= v->max_seq_len, FC_EINVAL,
               "%s: block table (%d entries of %d tokens) shorter than max_seq_len %d", who,
               v->table_stride, v->block_size, v->max_seq_len);
  }
  // 16-byte vector accesses: every stride must keep rows 16-byte aligned.
  const int64_t q = 16 / fc_elem_bytes(v->dtype);
  FC_REQUIRE(((uintptr_t)v->base & 15) == 0, FC_EINVAL, "%s: base not 16-byte aligned", who);
  FC_REQUIRE(v->stride_layer % q == 0 && v->stride_block % q == 0 && v->stride_batch % q == 0 &&
                 v->stride_token % q == 0 && v->stride_head % q == 0,
             FC_EINVAL, "%s: strides must be multiples of %lld elements", who, (long long)q);
  return FC_OK;
}
