// Which prefill tile serves a call, how it is planned (query rows per workgroup, key-range parts, scratch) and
// its launch.  Many query rows per kv head (r = Hq / Hkv heads times L new tokens): quantized caches take the
// pipelined tile of kvhip_attend_prefill_q.hpp, full-precision caches the kernel of kvhip_attend_prefill_fp.hip.
#include <cstdlib>

#include "kvhip_mask.hpp"

namespace kvhip {

constexpr int BN = 32;  // key slots per tile (both kernels)

bool attend_prefill_supported(const AttendArgs &a) {
    const Store &s = a.st;
    if (s.dtype != KVHIP_F16 && s.dtype != KVHIP_BF16) return false;
    if (s.bits != 0) return attend_prefill_q_supported(a);
    // full precision: keys of 192 with values of 128 (the multi-head latent attention models), or one head size;
    // 80 and 96 at every row count (no decode kernel is built for them)
    if (s.Dk == 192 && s.Dv == 128) return true;
    if (s.Dk != s.Dv) return false;
    return s.Dk == 64 || s.Dk == 80 || s.Dk == 96 || s.Dk == 128 || s.Dk == 256;
}

// A prompt chunk over a quantized cache converts every cached row once per workgroup that reads it.  With many query
// rows per kv head it is cheaper to convert the rows once for all of them: the cache is dequantized into scratch
// pages of its dtype and the full-precision tile, whose loop has no conversions, runs over those.  The scratch costs
// 2 (Dk + Dv) bytes per cached row and kv head written and read again; the tile gains about a third of its time.
bool attend_prefill_dequant_first(const AttendArgs &a, bool always) {
    const Store &s = a.st;
    if (s.bits == 0 || (s.dtype != KVHIP_F16 && s.dtype != KVHIP_BF16)) return false;
    if (a.runs.n != 1 || a.runs.row0[0] != 0 || a.runs.phys0[0] != 0) return false;
    if (s.Dk % 8 != 0 || s.Dv % 8 != 0) return false;
    AttendArgs fp = a;
    fp.st.bits = 0;
    if (!attend_prefill_supported(fp)) return false;
    if (always) return true;
    // The conversion pass is a launch more and 2 (Dk + Dv) bytes per cached row and kv head written and read again,
    // the same for any number of query rows: what it buys grows with the rows per kv head that share a converted
    // key.  Per kv head both costs scale alike with batch and heads, so the bound is one on rows x keys x head
    // sizes: measured ahead by 5-40 % from 512 rows and rows x keys = 4 M at D 128 (2048 x 2048, 1024 x 4096,
    // 512 x 8192; B1 to B16) over 2048 keys and more, equal or behind below that (1024 x 2048: 44 against 40 us,
    // 2048 x 1024: 44 against 42, 4096 x 1024: 50 against 41,
    // B16 512 x 4096, where 256-row workgroups of the quantized tile fill the chip: 231 against 197) and with
    // fewer rows whatever the keys (B8, 256 x 8192: 185 against 141 us).
    const int R = (a.Hq / a.Hkv) * a.L;
    static const int min_rows = measure_knob("KVHIP_DEQUANT_FIRST_ROWS", 512);  // (timing builds only)
    return R >= min_rows && a.T >= 2048 && (double)R * a.T * (s.Dk + s.Dv) >= 1073741824.0;
}

// 128 query rows per workgroup reuse each staged tile twice as often as 64, and measured ahead of 64 rows on every
// grid from two such blocks per kv head up -- also where they leave the grid small, which key-range parts then fill
// (TFLOP/s of the call, 64 / 128 rows, fp16 D 128 32q/8kv causal: B1 512 x 8192 542 / 598, 512 x 32768 709 / 855,
// 1024 x 8192 590 / 714, 256 x 32768 643 / 754, B2 512 x 8192 603 / 712, B7 256 x 4096 547 / 695, B3 512 x 8192
// 693 / 708; D 64 B1 2048 x 8192 334 / 446; equal at 128 rows of 4 heads).
static bool prefill_wide(const AttendArgs &a) {
    const int R = (a.Hq / a.Hkv) * a.L;
    static const int forced = measure_knob("KVHIP_PREFILL_WIDE", -1);  // (timing builds only)
    if (forced >= 0) return forced != 0 && a.st.Dk <= 128;
    if (R < 256 || a.st.Dk > 128) return false;
    // Few keys (a prompt's first chunks): where 128-row workgroups would need key-range parts to fill the chip and
    // 64-row ones fill it without, the merge launch costs more than the wider tile gains (a single sequence's
    // 512 x 512: 22 against 35 us; 512 x 1024: 33 against 43; equal from 2048 keys).
    const size_t wide_wgs = (size_t)((R + 127) / 128) * a.st.BH, narrow_wgs = (size_t)((R + 63) / 64) * a.st.BH;
    if (a.T <= 1024 && wide_wgs < 512 && narrow_wgs >= 256) return false;
    return true;
}

// Query rows per workgroup.  The pipelined tile for quantized caches (kvhip_attend_prefill_q.hpp) takes 256 rows
// on 8 wavefronts at head size 128, one workgroup per CU, whenever that still gives every CU a workgroup: four
// times as many rows share each converted tile (B1, 2048 x 8192, 4 bits: 600 against 457 TFLOP/s).  Otherwise 128 or
// 64 rows on 4 wavefronts as above (quantized: 64; keys of 192 with values of 128: 128 rows on 8 wavefronts).
static int prefill_block_rows(const AttendArgs &a) {
    const int R = (a.Hq / a.Hkv) * a.L;
    if (a.st.bits != 0) {
        static const int forced = measure_knob("KVHIP_PREFILL_ROWS", 0);  // (timing builds only)
        if (forced == 64 || (forced == 128 && a.st.Dk == 192) || (forced == 256 && a.st.Dk == 128 && (a.st.bits == 4 || a.st.bits == 8))) return forced;
        // (head size 64 measured faster on 64 rows: 363 / 393 against 340 / 362 TFLOP/s at 8 / 4 bits, B4 2048 x 4096)
        if ((a.st.bits == 4 || a.st.bits == 8) && a.st.Dk == 128) {
            // 256 rows need a workgroup for every CU.  Under a causal or window mask the query blocks differ in work and a
            // CU holds one such workgroup at a time, so beyond a single round the gain depends on the shape (4-bit, B1, 8 kv
            // heads, TFLOP/s on 64 / 256 rows: 2048 x 4096 411 / 483, 2048 x 8192 457 / 600, 8192 x 8192 563 / 617,
            // 4096 x 8192 543 / 532, but 4096 x 4096 457 / 384 and B4 2048 x 2048 435 / 362): one round, or long sequences
            const size_t wgs = (size_t)((R + 255) / 256) * a.st.BH;
            if (wgs >= 256 && (a.mask.mode == KVHIP_MASK_NONE || wgs <= 320 || a.T >= 8192)) return 256;
        }
        // keys of 192 with values of 128: 128 rows on 8 wavefronts (head sizes 96 / 128 / 256 measured 4-20 % slower on it)
        return (a.st.Dk == 192 && (size_t)((R + 127) / 128) * a.st.BH >= 256) ? 128 : 64;
    }
    return prefill_wide(a) ? 128 : 64;
}

// Key-range parts per query block: only when the grid would leave most CUs without a
// second workgroup, and only while the partials stay small.
static int prefill_splits(const AttendArgs &a) {
    const int R = (a.Hq / a.Hkv) * a.L;
    const int bm = prefill_block_rows(a);
    if (a.st.bits != 0 && bm > 64) return 1;  // (chosen only when the grid fills the chip)
    const size_t wgs = (size_t)((R + bm - 1) / bm) * a.st.BH;
    // (few keys and a workgroup per CU: see prefill_wide; the quantized tile likewise -- a single sequence's 512 x 512
    // 4-bit chunk 33 -> 30 us undivided, 512 x 1024 at 8 bits 55 -> 47 us, at 4 bits 47 either way)
    if (a.T <= 1024 && wgs >= 256) return 1;
    // as many workgroups as are resident at once: three per CU, two at D = 256 (LDS) and for 128-row workgroups
    // (registers) -- a part more than that starts a second round that leaves half the CUs idle
    static const int forced = measure_knob("KVHIP_PREFILL_TARGET", 0);  // (timing builds only)
    const int target = forced > 0 ? forced : ((a.st.Dk >= 256 || (a.st.bits == 0 && bm == 128)) ? 512 : 768);
    int n = (int)(target / (wgs ? wgs : 1));
    const int tiles = (a.slots + BN - 1) / BN;
    if (n > tiles / 8) n = tiles / 8;
    // (a multi-token step or a short chunk of a few sequences -- up to 4096 query rows in all -- is a grid of a
    // handful of workgroups: up to 64 parts instead of 8, merged by the decode path's many-part kernel.  A
    // single sequence, 32q/8kv, 5 new tokens: over 8192 keys 43 -> 18 us at 4 bits and 31 -> 15 us in float16, over
    // 32768 keys 152 -> 31 us and 97 -> 28 us; 32 new tokens over 32768 keys 154 -> 50 us and 97 -> 39 us)
    const int cap = (size_t)R * a.st.BH <= 4096 ? 64 : 8;  // (the many-part merge takes a workgroup per query row)
    if (n > cap) n = cap;
    if (n < 2) return 1;
    const size_t per_part = (size_t)a.st.BH * R * (a.st.Dv + 2) * sizeof(float);
    if (per_part * n > ((size_t)256 << 20)) return 1;
    // a caller with a fixed amount of scratch: fewer parts until they fit (one part has no partials)
    while (a.workspace_cap && n > 1 && per_part * n > a.workspace_cap) --n;
    return n;
}

size_t attend_prefill_workspace(const AttendArgs &a) {
    const int n = prefill_splits(a);
    if (n <= 1) return 0;
    return (size_t)a.st.BH * n * (a.Hq / a.Hkv) * a.L * (a.st.Dv + 2) * sizeof(float);
}

hipError_t launch_attend_prefill(const AttendArgs &a, hipStream_t s) {
    const Store &st = a.st;
    const int R = (a.Hq / a.Hkv) * a.L;
    // 128 query rows per workgroup reuse each staged tile twice as often; 64 rows are used
    // when that would leave the grid too small to fill 256 CUs twice over
    const int bm = prefill_block_rows(a);
    const bool wide = bm == 128;
    const int nsplit = prefill_splits(a);
    if (st.bits != 0) {
        profile_mark(s, true);
        hipError_t e = launch_attend_prefill_q(a, nsplit, bm, s);
        profile_mark(s, false);
        if (e != hipSuccess) return e;
    } else {
        // full-precision caches have their own double-buffered kernel
        profile_mark(s, true);
        hipError_t e = launch_attend_prefill_fp(a, nsplit, wide, s);
        profile_mark(s, false);
        if (e != hipSuccess) return e;
    }
    if (nsplit > 1) {
        hipError_t e = launch_combine(a, nsplit, R, s);
        if (e != hipSuccess) return e;
    }
    return hipGetLastError();
}

}  // namespace kvhip
