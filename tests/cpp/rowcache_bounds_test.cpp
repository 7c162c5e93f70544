// Which bytes the shifted row accesses touch (blackforge_amd/csrc/rowcache.hpp: RowCache::issueShifted / maskShifted /
// storeShifted, the accesses of the cross-entropy kernels on rows of any length and alignment), checked on the CPU.
//
// RowCache itself is compiled here, for the host, over accessors that check every address: a read must lie between the
// tensor's first byte rounded DOWN to the boundary the caller chose (16 bytes, or 128 for tensors that start on a
// 128-byte line) and its last byte rounded UP to 16 bytes; a write must lie inside the tensor.  The tensors sit in a
// larger buffer whose surroundings hold a sentinel, and a row loaded and stored again must come out exactly as it went
// in (which pins the masks: one wrong slot would copy a neighbour's element or the fill value).
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#define BF_ROWCACHE_HOST_MODEL
#define __device__
#define __forceinline__ inline

namespace bf {
struct float4v { float x, y, z, w; };
struct uint2v { unsigned x, y; };
struct OpSum {};
struct OpMaxF {};
inline float waveMax(float v) { return v; }
template <typename T, typename Op> T blockReduce(T v, T, Op, T*) { return v; }
template <typename T> T __shfl_xor(T v, int, int) { return v; }
inline unsigned short toBf16Bits(float) { return 0; }

struct Window { uintptr_t readLo, readHi, writeLo, writeHi; };
Window g_window;
long g_violations = 0, g_reads = 0, g_writes = 0;
inline void checkRead(const void* p, size_t n) {
    const uintptr_t a = reinterpret_cast<uintptr_t>(p);
    ++g_reads;
    if (a < g_window.readLo || a + n > g_window.readHi) ++g_violations;
}
inline void checkWrite(const void* p, size_t n) {
    const uintptr_t a = reinterpret_cast<uintptr_t>(p);
    ++g_writes;
    if (a < g_window.writeLo || a + n > g_window.writeHi) ++g_violations;
}
template <bool NT> float4v ldf4(const float* p) {
    checkRead(p, 16);
    if (reinterpret_cast<uintptr_t>(p) % 16 != 0) ++g_violations;   // a 16-byte access of these kernels is aligned
    float4v v;
    std::memcpy(&v, p, 16);
    return v;
}
template <bool NT> float ldf1(const float* p) { checkRead(p, 4); return *p; }
template <bool NT> void stf4(float* p, float4v v) {
    checkWrite(p, 16);
    if (reinterpret_cast<uintptr_t>(p) % 16 != 0) ++g_violations;
    std::memcpy(p, &v, 16);
}
template <bool NT> void stf1(float* p, float v) { checkWrite(p, 4); *p = v; }
template <bool NT> void stu2(void* p, uint2v v) { checkWrite(p, 8); std::memcpy(p, &v, 8); }
}  // namespace bf

#include "../../blackforge_amd/csrc/rowcache.hpp"

namespace {
int failures = 0;
void report(bool ok, const char* what, size_t rows, size_t features, int group, int maxe, unsigned mask, size_t offsetBytes) {
    if (!ok) ++failures;
    std::printf("[%s] %s: %zu rows of %zu, group %d x %d registers, boundary %u bytes, tensor %zu bytes into a line\n", ok ? "  OK  " : " FAIL ",
                what, rows, features, group, maxe, 4 * (mask + 1), offsetBytes);
}

// A tensor [rows, features] that starts offsetBytes after a 128-byte line, copied row by row through a shifted load
// and a shifted store, as the cross-entropy kernel reads logits and writes gradients.
template <int G, int MAXE>
void copyThroughRowCache(size_t rows, size_t features, unsigned mask, size_t offsetBytes) {
    using Row = bf::RowCache<G, MAXE, 4>;
    constexpr float kSentinel = -12345.5f;
    if (features + mask > size_t(G) * MAXE) {   // the launcher's own condition for a plan (loss.hip)
        report(false, "the row with its extra slots fits the group's registers", rows, features, G, MAXE, mask, offsetBytes);
        return;
    }
    const size_t count = rows * features, guard = 256;   // floats on either side
    std::vector<float> srcBuf(count + 2 * guard + 64, kSentinel), dstBuf(count + 2 * guard + 64, kSentinel);
    auto place = [&](std::vector<float>& buf) {
        uintptr_t a = reinterpret_cast<uintptr_t>(buf.data() + guard);
        a = (a + 127) / 128 * 128 + offsetBytes;
        return reinterpret_cast<float*>(a);
    };
    float* src = place(srcBuf);
    float* dst = place(dstBuf);
    for (size_t i = 0; i < count; ++i) src[i] = float(i % 8191) + 0.25f;
    const uintptr_t boundary = 4 * (mask + 1);
    const uintptr_t first = reinterpret_cast<uintptr_t>(src), end = first + count * 4;
    bf::g_window = {first / boundary * boundary, (end + 15) / 16 * 16, reinterpret_cast<uintptr_t>(dst), reinterpret_cast<uintptr_t>(dst) + count * 4};
    const long before = bf::g_violations;
    for (size_t r = 0; r < rows; ++r) {
        const float* row = src + r * features;
        float* out = dst + r * features;
        const int shift = Row::shiftOf(row, mask);
        if (shift != Row::shiftOf(out, mask)) { report(false, "source and destination rows share their offset", rows, features, G, MAXE, mask, offsetBytes); return; }
        for (int t = 0; t < G; ++t) {
            Row c;
            c.loadShifted(row, features, t, -INFINITY, shift);
            // every slot outside the row must hold the fill value, every slot inside it the row's element
            for (int it = 0; it < Row::kIters; ++it)
                for (int j = 0; j < 4; ++j) {
                    const long e = long(it * G + t) * 4 + j - shift;
                    const float expect = (e >= 0 && e < long(features)) ? row[e] : -INFINITY;
                    if (c.r[it * 4 + j] != expect) ++bf::g_violations;
                }
            c.storeShifted(out, features, t, shift);
        }
    }
    bool ok = bf::g_violations == before;
    for (size_t i = 0; i < count && ok; ++i) ok = dst[i] == src[i];
    const float* dlo = dstBuf.data();   // nothing outside the tensor was written
    for (const float* p = dlo; p < dst && ok; ++p) ok = *p == kSentinel;
    for (const float* p = dst + count; p < dlo + dstBuf.size() && ok; ++p) ok = *p == kSentinel;
    report(ok, "shifted rows stay inside their tensor and come out as they went in", rows, features, G, MAXE, mask, offsetBytes);
}
}  // namespace

int main() {
    // the plans of the cross-entropy launcher (loss.hip): a wavefront, a 256-thread block or a 1024-thread block per row;
    // the 128-byte boundary only with 1024 threads, tensors that start on a line and rows with room for the 31 extra slots
    for (size_t offset : {size_t(0), size_t(4), size_t(8), size_t(12), size_t(64), size_t(100)}) {
        copyThroughRowCache<64, 4>(5, 33, 3u, offset);
        copyThroughRowCache<64, 16>(3, 1003, 3u, offset);
        copyThroughRowCache<64, 4>(7, 1, 3u, offset);
        copyThroughRowCache<256, 32>(3, 4100 + 1, 3u, offset);
        copyThroughRowCache<256, 8>(4, 2045, 3u, offset);   // the longest row this plan serves: 2045 + 3 slots = 256 x 8
        copyThroughRowCache<1024, 52>(2, 50257, 3u, offset);
        copyThroughRowCache<1024, 32>(3, 32001, 3u, offset);
    }
    copyThroughRowCache<1024, 52>(3, 50257, 31u, 0);
    copyThroughRowCache<1024, 52>(2, 53248 - 31, 31u, 0);   // the longest row the 128-byte boundary serves
    copyThroughRowCache<1024, 32>(5, 32001, 31u, 0);
    copyThroughRowCache<1024, 16>(4, 9999, 31u, 0);
    copyThroughRowCache<1024, 52>(1, 50257, 31u, 0);         // a single row: nothing before it, nothing after it
    std::printf("%ld reads and %ld writes checked, %d failure(s)\n", bf::g_reads, bf::g_writes, failures);
    return failures == 0 ? 0 : 1;
}
