// Environment-driven configuration of the training-side plugin, read once.
// Restates pytorch/torch_col/csrc/config.cc:49-147 (same variable names, same defaults,
// same derived flags).
#pragma once

#include <string>

namespace tch {
namespace host {

struct Config {
  bool configured = false;
  int train_rank = 0;
  int train_world_size = 1;
  bool use_shared_tensor = false;           // COLTRAIN_USE_SHARED_TENSOR
  double shared_tensor_pool_gb = 12.0;      // COLTRAIN_SHARED_TENSOR_POOL_GB
  bool has_colocated_infer_server = false;  // COLTRAIN_HAS_INFER_SERVER
  bool has_shared_tensor_server = false;    // COLTRAIN_HAS_SHARED_TENSOR_SERVER
  bool colocate_use_xsched = false;         // COLTRAIN_USE_XSCHED
  bool kill_batch_on_recv = false;          // hook mode xsched-sync2 AND xsched
  bool dynamic_sm_partition = false;        // COLTRAIN_DYNAMIC_SM_PARTITION AND xsched
  std::string colocate_ctrl_hook_mode = "none";  // COLTRAIN_HOOK_MODE
  std::string colocate_train_mode = "normal";    // COLTRAIN_MODE
  bool is_colocate_l1 = false;
  bool is_colocate_l2 = false;
  bool release_interm_memory_by_grad_fn = false;
  bool release_interm_memory_by_tagging = true;
  bool use_fbward_hook = true;
  std::string train_profile_log_path;  // COLTRAIN_PROFILE_LOG_PATH
  bool log_all = false, log_dynamic_batch = false, log_control_stub = false;
};

Config& config();
// (re)reads the environment unless already configured; `force` re-reads anyway (tests).
void init_config(int train_rank, int train_world_size, bool force);
// hook mode / train mode enums as the reference numbers them (cython/util_cls.pxi:7-38)
int hook_mode_code(const std::string& s);   // none 0, sync 1, xsched-sync 2, xsched-sync2 3; -1 unknown
int train_mode_code(const std::string& s);  // normal 0, colocate-l1 1, colocate-l2 2, taskswitch-l1 3, -l2 4, -l3 5, -l0 6

}  // namespace host
}  // namespace tch
