// Host stand-in for daceml_amd/csrc/lds_ops.h (same names, same meaning) over the fibre scheduler of emu.h.
// TEST INFRASTRUCTURE ONLY.
#pragma once

#include "common.h"

namespace dml {

typedef _Float16 half4v __attribute__((ext_vector_type(4)));

// LDS "addresses" are byte offsets into emu::g_lds
inline uint32_t lds_addr(const void* p) { return (uint32_t)((const char*)p - emu::g_lds); }

// 16 bytes per lane, global -> LDS: lane l's piece lands at lds_dst + 16 * l
inline void lds_dma16(const _Float16* gptr, char* lds_dst) {
    emu::dma_issue(gptr, lds_addr(lds_dst) + 16 * (threadIdx.x & 63), 16);
}

template <int OFFSET>
inline half8 lds_read_b128(uint32_t addr) {
    half8 v;
    memcpy(&v, emu::g_lds + addr + OFFSET, 16);
    return v;
}

// ds_read_b64_tr_b16: within each group of 16 lanes, lane s supplies the address of four consecutive 16-bit elements;
// the 16 x 4 elements form rows s / 4 (four lanes side by side make one row of 16); lane j receives element j of each
// of the four rows
template <int OFFSET>
inline half4v lds_read_tr16_b64(uint32_t addr) {
    const uint32_t mine = addr + OFFSET;
    const uint32_t* all = static_cast<const uint32_t*>(emu::wave_exchange(&mine, sizeof(mine)));
    const int lane = threadIdx.x & 63, group = lane & ~15, j = lane & 15;
    half4v v;
    for (int row = 0; row < 4; ++row) {
        const uint32_t a = all[group + row * 4 + j / 4];
        _Float16 e;
        memcpy(&e, emu::g_lds + a + 2 * (j % 4), 2);
        v[row] = e;
    }
    return v;
}

inline void global_store_b128_through(void* p, half8 v) { *static_cast<half8*>(p) = v; }

template <int N>
inline void wait_lgkm() {}

template <int VM>
inline void wait_vm_lgkm0() { emu::dma_wait(VM); }

}  // namespace dml
