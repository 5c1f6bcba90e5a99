#include "fa_common.hpp"
#include "launch.hpp"
namespace fa {
int bwd_dkv_bf16_d128(const BwdArgs&, hipStream_t) { return set_error(FLEXATTN_ENOTSUP, "bf16 dkv not built yet"); }
void bwd_dkv_bf16_d128_tile(int* bq, int* bk) { *bq = 64; *bk = 128; }
}
