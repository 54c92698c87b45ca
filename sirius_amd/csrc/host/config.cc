#include "config.h"

#include <stdlib.h>
#include <unistd.h>

#include <iostream>
#include <sstream>

namespace tch {
namespace host {

namespace {
Config g_config;

bool env_is_one(const char* name) {
  const char* v = getenv(name);
  return v != nullptr && std::string(v) == "1";
}
std::string env_or(const char* name, const char* dflt) {
  const char* v = getenv(name);
  return v ? std::string(v) : std::string(dflt);
}
}  // namespace

Config& config() { return g_config; }

void init_config(int train_rank, int train_world_size, bool force) {
  Config& c = g_config;
  if (c.configured && !force) return;
  c = Config();
  c.train_rank = train_rank;
  c.train_world_size = train_world_size;
  c.use_shared_tensor = env_is_one("COLTRAIN_USE_SHARED_TENSOR");
  c.colocate_use_xsched = env_is_one("COLTRAIN_USE_XSCHED");
  c.has_colocated_infer_server = env_is_one("COLTRAIN_HAS_INFER_SERVER");
  c.has_shared_tensor_server = env_is_one("COLTRAIN_HAS_SHARED_TENSOR_SERVER");
  c.dynamic_sm_partition = env_is_one("COLTRAIN_DYNAMIC_SM_PARTITION") && c.colocate_use_xsched;
  c.colocate_ctrl_hook_mode = env_or("COLTRAIN_HOOK_MODE", "none");
  c.colocate_train_mode = env_or("COLTRAIN_MODE", "normal");
  c.train_profile_log_path = env_or("COLTRAIN_PROFILE_LOG_PATH", "");
  c.is_colocate_l1 = c.colocate_train_mode == "colocate-l1";
  c.is_colocate_l2 = c.colocate_train_mode == "colocate-l2";
  c.log_all = env_is_one("COLTRAIN_LOG_ALL");
  c.log_dynamic_batch = c.log_all || env_is_one("COLTRAIN_LOG_DYNAMIC_BATCH");
  c.log_control_stub = c.log_all || env_is_one("COLTRAIN_LOG_CONTROL_STUB");
  // a kill on receipt needs the launch queue in front of the stream
  c.kill_batch_on_recv = c.colocate_ctrl_hook_mode == "xsched-sync2" && c.colocate_use_xsched;
  if (const char* gb = getenv("COLTRAIN_SHARED_TENSOR_POOL_GB")) c.shared_tensor_pool_gb = atof(gb);
  c.configured = true;
  if (c.log_all) {
    std::ostringstream ss;
    ss << "================ TORCH_COL CONFIG [Rank " << c.train_rank << " PID " << getpid() << "] ================\n"
       << "rank=" << c.train_rank << "|world_size=" << c.train_world_size << "\n"
       << "use_shared_tensor=" << c.use_shared_tensor << "\n"
       << "colocate_use_xsched=" << c.colocate_use_xsched << "\n"
       << "kill_batch_on_recv=" << c.kill_batch_on_recv << "\n"
       << "has_colocated_infer_server=" << c.has_colocated_infer_server << "\n"
       << "has_shared_tensor_server=" << c.has_shared_tensor_server << "\n"
       << "shared_tensor_pool_gb=" << c.shared_tensor_pool_gb << "\n"
       << "colocate_ctrl_hook_mode=" << c.colocate_ctrl_hook_mode << "\n"
       << "colocate_train_mode=" << c.colocate_train_mode << "\n"
       << "train_profile_log_path=" << c.train_profile_log_path << "\n";
    std::cerr << ss.str() << std::endl;
  }
}

int hook_mode_code(const std::string& s) {
  if (s == "none") return 0;
  if (s == "sync") return 1;
  if (s == "xsched-sync") return 2;
  if (s == "xsched-sync2") return 3;
  return -1;
}

int train_mode_code(const std::string& s) {
  if (s == "normal") return 0;
  if (s == "colocate-l1") return 1;
  if (s == "colocate-l2") return 2;
  if (s == "taskswitch-l1") return 3;
  if (s == "taskswitch-l2") return 4;
  if (s == "taskswitch-l3") return 5;
  if (s == "taskswitch-l0") return 6;
  return -1;
}

}  // namespace host
}  // namespace tch
