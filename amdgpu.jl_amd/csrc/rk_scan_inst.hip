// Instantiates the scan kernels for one element-type pair per object file
// (compiled several times with -DRK_INST=<n>).
#include "rk_scan_impl.hpp"

namespace rk {
#if RK_INST == 0
int32_t scan_f32(const ScanArgs& a) { return scan_typed<float, float>(a); }
#elif RK_INST == 1
int32_t scan_f64(const ScanArgs& a) { return scan_typed<double, double>(a); }
#elif RK_INST == 2
int32_t scan_i32(const ScanArgs& a) { return scan_typed<int32_t, int32_t>(a); }
#elif RK_INST == 3
int32_t scan_i64(const ScanArgs& a) { return scan_typed<int64_t, int64_t>(a); }
#elif RK_INST == 4
int32_t scan_u8_i64(const ScanArgs& a) { return scan_typed<uint8_t, int64_t>(a); }
#elif RK_INST == 5
int32_t scan_u8_i32(const ScanArgs& a) { return scan_typed<uint8_t, int32_t>(a); }
#elif RK_INST == 6
int32_t scan_u32(const ScanArgs& a) { return scan_typed<uint32_t, uint32_t>(a); }
#elif RK_INST == 7
int32_t scan_u64(const ScanArgs& a) { return scan_typed<uint64_t, uint64_t>(a); }
#elif RK_INST == 8
int32_t scan_i8(const ScanArgs& a) { return scan_typed<int8_t, int32_t, int8_t>(a); }
#elif RK_INST == 9
int32_t scan_u8(const ScanArgs& a) { return scan_typed<uint8_t, uint32_t, uint8_t>(a); }
#elif RK_INST == 10
int32_t scan_i16(const ScanArgs& a) { return scan_typed<int16_t, int32_t, int16_t>(a); }
#elif RK_INST == 11
int32_t scan_u16(const ScanArgs& a) { return scan_typed<uint16_t, uint32_t, uint16_t>(a); }
#elif RK_INST == 12
int32_t scan_f16(const ScanArgs& a) { return scan_typed<half_t, float, half_t>(a); }
#else
#error "RK_INST must be 0..12"
#endif
}  // namespace rk
