// Library-wide pieces of the C ABI: version, thread-local error string, shape queries, descriptor checks.
#include <string.h>

#include "abi_util.hpp"

namespace hyc {

char* error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

int make_chan_args(const hyc_desc* d, const RowGeom& g, ChanArgs* a, int* lpg) {
  int rc = chan_geom(g, d->group, lpg);
  if (rc) return rc;
  if (d->k < 0 || d->k > g.H || d->k > 65535) return fail(HYC_EINVAL, "k=%d out of range for H=%lld", d->k, (long long)g.H);
  if (!d->chan_plan) return fail(HYC_EFAULT, "channel mode needs chan_plan (from hyc_select_channels)");
  if (d->k > 0 && !d->chan_idx) return fail(HYC_EFAULT, "channel mode needs chan_idx (from hyc_select_channels) when k > 0");
  a->plan = d->chan_plan;
  a->idx = d->chan_idx;
  a->k = d->k;
  a->groups_per_row = (int)(g.H / d->group);
  a->chunk_to_group_shift = ilog2(*lpg);
  if (d->scale_rule != HYC_SCALE_RANGE && d->scale_rule != HYC_SCALE_ABSMAX)
    return fail(HYC_EINVAL, "scale_rule=%d: HYC_SCALE_RANGE (0) or HYC_SCALE_ABSMAX (1)", d->scale_rule);
  a->absmax = d->scale_rule == HYC_SCALE_ABSMAX;
  return HYC_OK;
}

int make_thr_args(const hyc_desc* d, const RowGeom& g, ThrArgs* a, bool* perchan) {
  if (!d->scale) return fail(HYC_EFAULT, "threshold mode needs a static scale");
  if (d->S <= 0) return fail(HYC_EINVAL, "threshold mode needs S (rows per batch element) > 0");
  if (d->scale_stride_channel == 1 && (d->scale_stride_token % 8) == 0 && aligned16(d->scale)) {
    *perchan = true;
  } else if (d->scale_stride_channel == 0) {
    *perchan = false;
  } else {
    return fail(HYC_ENOTSUP, "scale strides (%lld, %lld): per-tensor (0,0), per-token (1,0) and per-channel (0,1) are covered",
                (long long)d->scale_stride_token, (long long)d->scale_stride_channel);
  }
  if (d->rank < 0 || d->rank > 64) return fail(HYC_EINVAL, "rank=%d out of range (0..64)", d->rank);
  if (d->rank > 0) {
    if (!d->L || !d->R) return fail(HYC_EFAULT, "rank > 0 needs L and R");
    if (!aligned16(d->R)) return fail(HYC_EINVAL, "R must be 16-byte aligned");
  }
  a->thr = round_to_bf16(d->threshold);
  a->scale = static_cast<const uint16_t*>(d->scale);
  a->sst = d->scale_stride_token;
  a->ssc = d->scale_stride_channel;
  a->S = d->S;
  a->L = static_cast<const uint16_t*>(d->L);
  a->R = static_cast<const uint16_t*>(d->R);
  a->rank = d->rank;
  a->row_ptr = d->csr_row_ptr;
  a->cols = d->csr_cols;
  a->vals = static_cast<const uint16_t*>(d->csr_vals);
  (void)g;
  return HYC_OK;
}

}  // namespace hyc

using namespace hyc;

extern "C" {

int hyc_abi_version(void) { return HYC_ABI_VERSION; }

const char* hyc_last_error(void) { return error_buffer(); }

int hyc_check_shape(int64_t H, int32_t bits, int32_t group, int32_t mode) {
  RowGeom g;
  int rc = row_geom(H, bits, &g);
  if (rc) return rc;
  if (mode == HYC_MODE_CHANNEL) {
    int lpg;
    return chan_geom(g, group, &lpg);
  }
  if (mode == HYC_MODE_THRESHOLD || mode == HYC_MODE_DENSE) return HYC_OK;
  return fail(HYC_EINVAL, "mode=%d unknown", mode);
}

int64_t hyc_stored_row_bytes(int64_t H, int32_t bits) { return H * bits / 8; }

}  // extern "C"
