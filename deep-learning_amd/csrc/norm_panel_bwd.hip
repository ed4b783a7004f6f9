// placeholder until the backward panel kernel is written
#include "norm_panel_common.hpp"
namespace dlmi {
int panel_bwd_try(dlmi_ctx *, size_t, size_t, BwdCall const &, bool) { return 0; }
}  // namespace dlmi
