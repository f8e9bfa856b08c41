// Launch parameter blocks and internal launcher prototypes shared by the kernel
// translation units and the C ABI (fv_api.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fv {

struct FlashParams {
    const uint16_t* q;
    const uint16_t* k;
    const uint16_t* v;
    float* out_f32;
    uint16_t* out_bf16;
    int out_is_bf16;
    int sq, sk;
    float sl2;          // scale * log2(e)
    int nqt;            // query tiles per (batch, head)
    int total;          // bh * nqt
    int per_xcd;        // ceil(total / 8)
    int ft, win, sink;  // block-causal: block tokens, window blocks, sink blocks
};

}  // namespace fv

extern "C" hipError_t fv_internal_launch_flash(const fv::FlashParams* p, int causal,
                                               hipStream_t stream);
