#include "fa_common.hpp"
#include "launch.hpp"
namespace fa {
int bwd_dq_bf16_d128(const BwdArgs&, hipStream_t) { return set_error(FLEXATTN_ENOTSUP, "bf16 dq not built yet"); }
void bwd_dq_bf16_d128_tile(int* bq, int* bk) { *bq = 128; *bk = 64; }
}
