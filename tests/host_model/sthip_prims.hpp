// Host stand-in for strassen-triton_amd/csrc/sthip_prims.hpp (found first on the include path of the
// host build): the same functions, defined in kernel4_host.cpp.
#pragma once
namespace sthip {
void lds_dma16(const void* sbase, uint32_t voff, uint32_t lds_addr);
void lds_dma16_k(const void* sbase, uint32_t voff, uint32_t lds_addr, int k);
void lds_dma16_km(const void* sbase, uint32_t voff, uint32_t lds_addr, int k, uint32_t mask);
s16x4 lds_read_tr16_b64(const char* p);
void mfma16_step_f32(f32x4& acc, uint32_t a, uint32_t b);
template <class T> void mfma16_step(f32x4& acc, const u32x4& a, const u32x4& b);
void wave_exchange_point();
void gload16_6(f32x4& dst, const float* p);
inline void tie6(f32x4&) {}
}  // namespace sthip
