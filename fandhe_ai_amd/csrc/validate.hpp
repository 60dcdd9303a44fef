// Host-side checks shared by the paged KV entry points.
#pragma once

#include "runtime.hpp"

namespace fa {
fa_status paged_layout_check(const fa_paged_layout *l);
fa_status paged_args_check(const fa_paged_args *a);
uint64_t paged_kv_heads(const fa_paged_args *a);
}  // namespace fa
