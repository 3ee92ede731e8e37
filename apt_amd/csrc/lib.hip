// Library-wide state of libapt_hip.so: per-thread error text, ABI version and
// the tuning knobs the benchmark uses to compare kernel variants.
#include "common.hpp"

#include <cstring>

namespace apt {

char* last_error_buf() {
  static thread_local char buf[512] = {0};
  return buf;
}

static int g_sample_lanes = 0;
static int g_gather_rows = 0;
static int g_gather_max_blocks = 0;
static int g_fuse_mark = 1;
static int g_payload_bits = 0;

int tuning_sample_lanes() { return g_sample_lanes; }
int tuning_gather_rows() { return g_gather_rows; }
// Launch caps of the calling thread (the epoch driver's thread shapes its launches for co-residency); a
// process-wide knob, when set, wins.
static thread_local int t_sample_max_blocks = 0, t_gather_max_blocks = 0;
void set_thread_launch_caps(int sample_blocks, int gather_blocks) {
  t_sample_max_blocks = sample_blocks;
  t_gather_max_blocks = gather_blocks;
}
int tuning_gather_max_blocks() { return g_gather_max_blocks != 0 ? g_gather_max_blocks : t_gather_max_blocks; }
int tuning_fuse_mark() { return g_fuse_mark; }
int tuning_payload_bits() { return g_payload_bits; }
static int g_sample_max_blocks = 0;
int tuning_sample_max_blocks() { return g_sample_max_blocks != 0 ? g_sample_max_blocks : t_sample_max_blocks; }
static int g_sample_min_workgroups = 0;
int tuning_sample_min_workgroups() { return g_sample_min_workgroups; }
static int g_sample_direct_rows = 0;
int tuning_sample_direct_rows() { return g_sample_direct_rows; }
static int g_gather_vector_bytes = 0;
int tuning_gather_vector_bytes() { return g_gather_vector_bytes; }
static int g_gather_store_policy = 0;
int tuning_gather_store_policy() { return g_gather_store_policy; }
static int g_gather_wt_tail_mib = 0;
int tuning_gather_wt_tail_mib() { return g_gather_wt_tail_mib; }
static int g_relabel_lds = 1;
int tuning_relabel_lds() { return g_relabel_lds; }
static int g_block_fused_scan = 1;
int tuning_block_fused_scan() { return g_block_fused_scan; }

}  // namespace apt

extern "C" const char* apt_last_error(void) { return apt::last_error_buf(); }

extern "C" int apt_abi_version(void) { return APT_ABI_VERSION; }

extern "C" int apt_set_tuning(const char* key, int value) {
  if (key == nullptr) return apt::fail(APT_EINVAL, "apt_set_tuning: key is NULL");
  if (std::strcmp(key, "sample_lanes_per_row") == 0) {
    if (value != 0 && value != 8 && value != 16 && value != 32 && value != 64)
      return apt::fail(APT_EINVAL, "apt_set_tuning: sample_lanes_per_row must be 0, 8, 16, 32 or 64");
    apt::g_sample_lanes = value;
    return APT_OK;
  }
  if (std::strcmp(key, "gather_rows_in_flight") == 0) {
    if (value != 0 && value != 1 && value != 2 && value != 4 && value != 8)
      return apt::fail(APT_EINVAL, "apt_set_tuning: gather_rows_in_flight must be 0, 1, 2, 4 or 8");
    apt::g_gather_rows = value;
    return APT_OK;
  }
  if (std::strcmp(key, "minibatch_payload_bits") == 0) {
    if (value < 0 || value > 31) return apt::fail(APT_EINVAL, "apt_set_tuning: minibatch_payload_bits must be 0..31");
    apt::g_payload_bits = value;
    return APT_OK;
  }
  if (std::strcmp(key, "minibatch_fuse_mark") == 0) {
    apt::g_fuse_mark = value != 0;
    return APT_OK;
  }
  if (std::strcmp(key, "sample_max_blocks") == 0) {
    if (value < 0) return apt::fail(APT_EINVAL, "apt_set_tuning: sample_max_blocks must be >= 0");
    apt::g_sample_max_blocks = value;
    return APT_OK;
  }
  if (std::strcmp(key, "sample_min_workgroups") == 0) {
    if (value < 0) return apt::fail(APT_EINVAL, "apt_set_tuning: sample_min_workgroups must be >= 0");
    apt::g_sample_min_workgroups = value;
    return APT_OK;
  }
  if (std::strcmp(key, "sample_direct_rows") == 0) {
    if (value != 0 && value != 1 && value != 2 && value != 4)
      return apt::fail(APT_EINVAL, "apt_set_tuning: sample_direct_rows must be 0, 1, 2 or 4");
    apt::g_sample_direct_rows = value;
    return APT_OK;
  }
  if (std::strcmp(key, "gather_vector_bytes") == 0) {
    if (value != 0 && value != 2 && value != 4 && value != 8 && value != 16)
      return apt::fail(APT_EINVAL, "apt_set_tuning: gather_vector_bytes must be 0, 2, 4, 8 or 16");
    apt::g_gather_vector_bytes = value;
    return APT_OK;
  }
  if (std::strcmp(key, "gather_store_policy") == 0) {
    if (value < 0 || value > 3)
      return apt::fail(APT_EINVAL, "apt_set_tuning: gather_store_policy must be 0 (by output size), 1 (non-temporal), "
                                   "2 (plain) or 3 (write-through)");
    apt::g_gather_store_policy = value;
    return APT_OK;
  }
  if (std::strcmp(key, "gather_wt_tail_mib") == 0) {
    APT_REQUIRE(value >= 0 && value <= 1024, APT_EINVAL, "apt_set_tuning: gather_wt_tail_mib must be in [0, 1024]");
    apt::g_gather_wt_tail_mib = value;
    return APT_OK;
  }
  if (std::strcmp(key, "relabel_lds") == 0) {
    apt::g_relabel_lds = value != 0;
    return APT_OK;
  }
  if (std::strcmp(key, "block_fused_scan") == 0) {
    apt::g_block_fused_scan = value != 0;
    return APT_OK;
  }
  if (std::strcmp(key, "gather_max_blocks") == 0) {
    if (value < 0) return apt::fail(APT_EINVAL, "apt_set_tuning: gather_max_blocks must be >= 0");
    apt::g_gather_max_blocks = value;
    return APT_OK;
  }
  return apt::fail(APT_EINVAL, "apt_set_tuning: unknown key '%s'", key);
}
