// Instantiates the reduction kernels for one element-type pair per object file
// (compiled several times with -DRK_INST=<n> so the instantiations build in parallel).
#include "rk_reduce_impl.hpp"

namespace rk {
#if RK_INST == 0
int32_t mapreduce_f32(const MapreduceArgs& a) { return mapreduce_typed<float, float>(a); }
int32_t findminmax_f32(const FindArgs& a) { return findminmax_typed<float>(a); }
int32_t mapreduce_prog_f32(const MapreduceArgs& a) { return mapreduce_prog<float, float>(a); }
int32_t mapreduce_prog_f32_i64(const MapreduceArgs& a) { return mapreduce_prog<float, int64_t, true>(a); }
#elif RK_INST == 1
int32_t mapreduce_f64(const MapreduceArgs& a) { return mapreduce_typed<double, double>(a); }
int32_t findminmax_f64(const FindArgs& a) { return findminmax_typed<double>(a); }
int32_t mapreduce_prog_f64(const MapreduceArgs& a) { return mapreduce_prog<double, double>(a); }
int32_t mapreduce_prog_f64_i64(const MapreduceArgs& a) { return mapreduce_prog<double, int64_t, true>(a); }
#elif RK_INST == 2
int32_t mapreduce_i32(const MapreduceArgs& a) { return mapreduce_typed<int32_t, int32_t>(a); }
int32_t findminmax_i32(const FindArgs& a) { return findminmax_typed<int32_t>(a); }
int32_t mapreduce_prog_i32(const MapreduceArgs& a) { return mapreduce_prog<int32_t, int32_t>(a); }
#elif RK_INST == 3
int32_t mapreduce_i64(const MapreduceArgs& a) { return mapreduce_typed<int64_t, int64_t>(a); }
int32_t findminmax_i64(const FindArgs& a) { return findminmax_typed<int64_t>(a); }
int32_t mapreduce_prog_i64(const MapreduceArgs& a) { return mapreduce_prog<int64_t, int64_t>(a); }
#elif RK_INST == 4
int32_t mapreduce_i32_i64(const MapreduceArgs& a) { return mapreduce_typed<int32_t, int64_t>(a); }
int32_t mapreduce_prog_i32_i64(const MapreduceArgs& a) { return mapreduce_prog<int32_t, int64_t>(a); }
#elif RK_INST == 5
int32_t mapreduce_u8_i64(const MapreduceArgs& a) { return mapreduce_typed<uint8_t, int64_t>(a); }
int32_t mapreduce_prog_u8_i64(const MapreduceArgs& a) { return mapreduce_prog<uint8_t, int64_t>(a); }
#elif RK_INST == 6
int32_t mapreduce_u8(const MapreduceArgs& a) { return mapreduce_typed<uint8_t, uint8_t>(a); }      // any / all of Bool arrays
int32_t findminmax_u8(const FindArgs& a) { return findminmax_typed<uint8_t>(a); }                   // findfirst of Bool arrays
#elif RK_INST == 7
int32_t mapreduce_u32(const MapreduceArgs& a) { return mapreduce_typed<uint32_t, uint32_t>(a); }
int32_t mapreduce_u32_u64(const MapreduceArgs& a) { return mapreduce_typed<uint32_t, uint64_t>(a); }   // add_sum widens UInt32 to UInt64
int32_t findminmax_u32(const FindArgs& a) { return findminmax_typed<uint32_t>(a); }
#elif RK_INST == 8
int32_t mapreduce_u64(const MapreduceArgs& a) { return mapreduce_typed<uint64_t, uint64_t>(a); }
int32_t findminmax_u64(const FindArgs& a) { return findminmax_typed<uint64_t>(a); }
#elif RK_INST == 9
// Float16 arrays: f in Float16 (abs2 rounds like Julia's), accumulation in Float32, one rounding at the end
int32_t mapreduce_f16(const MapreduceArgs& a) { return mapreduce_typed<half_t, float, half_t>(a); }
int32_t findminmax_f16(const FindArgs& a) { return findminmax_typed<half_t>(a); }
#elif RK_INST == 10
// narrow integers: sums and products in the 64-bit type Base.add_sum / mul_prod widen them to, max / min in their own
int32_t mapreduce_i8_i64(const MapreduceArgs& a) { return mapreduce_typed<int8_t, int64_t>(a); }
int32_t mapreduce_i8(const MapreduceArgs& a) { return mapreduce_typed<int8_t, int8_t>(a); }
int32_t findminmax_i8(const FindArgs& a) { return findminmax_typed<int8_t>(a); }
#elif RK_INST == 11
int32_t mapreduce_i16_i64(const MapreduceArgs& a) { return mapreduce_typed<int16_t, int64_t>(a); }
int32_t mapreduce_i16(const MapreduceArgs& a) { return mapreduce_typed<int16_t, int16_t>(a); }
int32_t findminmax_i16(const FindArgs& a) { return findminmax_typed<int16_t>(a); }
#elif RK_INST == 12
int32_t mapreduce_u16_u64(const MapreduceArgs& a) { return mapreduce_typed<uint16_t, uint64_t>(a); }
int32_t mapreduce_u16(const MapreduceArgs& a) { return mapreduce_typed<uint16_t, uint16_t>(a); }
int32_t findminmax_u16(const FindArgs& a) { return findminmax_typed<uint16_t>(a); }
#else
#error "RK_INST must be 0..12"
#endif
}  // namespace rk
