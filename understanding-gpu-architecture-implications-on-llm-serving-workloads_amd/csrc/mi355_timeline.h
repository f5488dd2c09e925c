// Profiling build only (compiled with -DMI355_TIMELINE into libmi355_serving_timeline.so; the product library carries none
// of this): a kernel stamps the 100 MHz wall clock and the shader cycle counter at a few points per workgroup and leaves
// them in a device array that `bench.py --timeline` reads back. Each kernel source that uses it owns its array (device
// symbols are per translation unit) and exports a reader.
#pragma once
#ifdef MI355_TIMELINE
namespace mi355 {
namespace timeline {
constexpr int kSlots = 8;               // 64-bit values per workgroup
constexpr int kMaxWorkgroups = 4096;    // workgroups beyond this leave no record
// The wait is part of the same asm statement, so the value is valid when the statement ends (the compiler does not track
// the scalar memory counter of inline asm). Scalar loads only: nothing is written through the scalar cache.
__device__ __forceinline__ unsigned long long wall_clock() {
    unsigned long long t;
    asm volatile("s_memrealtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(t));
    return t;
}
__device__ __forceinline__ unsigned long long shader_cycles() {
    unsigned long long t;
    asm volatile("s_memtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(t));
    return t;
}
}  // namespace timeline
}  // namespace mi355
#define MI355_TL(...) __VA_ARGS__
#else
#define MI355_TL(...)
#endif
