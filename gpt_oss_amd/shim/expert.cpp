// Takes the place of the reference's getp-csrc/expert.cpp on one GPU, so that an
// unmodified getp-csrc/getp_run.cpp (which does `#include "expert.cpp"`,
// getp_run.cpp:4) builds against libmi355_moe:
//
//   mv getp-csrc/expert.cpp getp-csrc/expert_ref.cpp
//   cp <this file> getp-csrc/expert.cpp
//   hipcc ... -I<repo>/include -I<repo>/gpt_oss_amd/shim run.cpp tokenizer.cpp
//         -L<repo>/gpt_oss_amd -lmi355_moe
//
// The reference's file also holds two functions that are not part of the MoE
// layer and that getp_run.cpp calls (build_rope_tables, expert.cpp:439, used at
// getp_run.cpp:78; ensure_kv_cache_capacity, expert.cpp:497, used at
// getp_run.cpp:309 and :510).  They stay the reference's: its file is included
// here under its new name, with its four expert-parallel entry points renamed
// out of the way, and those four names are then defined by the shim on top of
// the C-ABI (include/moe_abi.h).
#define warm_up_ep ref_warm_up_ep
#define init_device_context_ep ref_init_device_context_ep
#define gpu_forward_device_batch_ep ref_gpu_forward_device_batch_ep
#define cleanup_device_context_ep ref_cleanup_device_context_ep
#include "expert_ref.cpp"
#undef warm_up_ep
#undef init_device_context_ep
#undef gpu_forward_device_batch_ep
#undef cleanup_device_context_ep

#define MI355_MOE_REPLACE_EP
#include "expert_mi355.hpp"
