// The static tiling table of the fused kernels: which (D, WAVES, UTW, KW) are compiled for each
// (gate-row count, storage type), forward and backward.  Replaces the reference's constraint
// solver + JIT bisection (flashrnn/flashrnn/flashrnn.py:429-589, cuda_init_parametric.py:92-358).
//
// X(D, VARIANT, WAVES, UTW, KW, MTR):  D = 16 * UTW * WAVES * KW;  MTR = the largest batch tile (4, 8 or 16 rows)
// this tiling is compiled for: taller tiles keep more state per lane, and where that would spill registers to
// scratch memory the tile height stops below (a large batch then runs as more groups, in several launches if
// the workgroups of a head wait for each other).  No compiled kernel uses scratch memory; a test checks the
// compiler's resource report of every instantiation.
//   R registers per lane = UTW * G_r * D / 8 (bf16) or UTW * G_r * D / 4 (f32); a workgroup of
//   4 waves (one per SIMD) may use up to 512 VGPRs per lane, one of 8 waves 256, of 16 waves 128.
// VARIANT 0 is the default.  VARIANT 2, where a head dim has one, spreads the head over more workgroups: it is
// used instead of the default while every workgroup of the call still gets a compute unit of its own with 4-row
// batch tiles (measured faster there, slower once the device is full).  To try another tiling add an
// X(D, 1, ...) entry and run with FRNN_FUSED_VARIANT=1.  The alternatives that were measured and lost (4 waves x 2 tiles for
// D = 128, 2 x 8 waves or 8 x 2 waves for D = 256, ...) are not compiled in.
// Forward and backward tile independently (the gate cache layout does not depend on the plan).
#pragma once

namespace frnn {
struct Plan {
  int D, variant, waves, utw, kw, max_tr;
  int cooperative = 0;  // host side only: launch the kernel as a cooperative one (see fused_*_tu.hip)
  int recompute = 0;    // host side only: the reverse kernel of recompute mode
};

// Resident operand of the forward product: a wave holds UTW*G_r*KS fragments of R.  When they alone
// would take more than 400 of the 512 registers a wave has at one wave per SIMD (LSTM D = 1024: all
// 512), those of the last RLK k-steps live in LDS instead (as many as bring the rest down to 352, and
// as fit beside the two h buffers) and are read back one k-step ahead as the A operand of their MFMAs.
constexpr int fwd_lds_ksteps(int GR, int D, int WAVES, int UTW, int esize) {
  const int KM = esize == 4 ? 4 : 32, FR = esize == 4 ? 1 : 4, FRB = esize == 4 ? 4 : 16;
  const int KS = D / KM, per = UTW * GR * FR, regs = per * KS;
  if (!(WAVES <= 4 && regs > 336)) return 0;
  const int want = (regs - 320 + per - 1) / per;
  const int room = (160 * 1024 - 2 * 16 * D * esize - 1024) / (WAVES * UTW * GR * 64 * FRB);
  return want < room ? want : room;
}

// Forward kernel, fp32 at 4-row tiles, cells with 3 or 4 recurrent gates: the product runs on v_mfma_f32_4x4x1_16B_f32
// (see the kernel), when the whole operand, D registers per tile in that form, fits the registers of a wave
// (workgroups of up to 4 waves: 512 registers each).
// Heads from 384 units on: the four waves of a workgroup pair up over two tiles, each wave of a pair keeps R for one half
// of k (D / 2 registers) and multiplies it with that half of h; the second wave hands its partial sums to the first
// through LDS, which alone does the gate math of the tile.  D = 16 * (WAVES / 2) * KW for these tilings.
// The same split for the 16-bit kernels of the 4-gate cells at D = 1024 (16x16x32 form: a tile of R is 512 registers, with
// the split 256 per wave, nothing of it in LDS, and room for the working sets of the 8- and 16-row tiles): the second
// wave hands over its G_r accumulators.
// fp32 heads beyond 512 units: all four waves share one tile, a quarter of k each (D / 4 registers), and three of them hand
// their sums over; D = 16 * KW (D = 640, 768, 1024: 40, 48, 64 workgroups per head), more than the 32 compute units of an XCD: such a group
// spreads over the device (decode_block) and exchanges at agent scope.
constexpr int fwd_k_split(int GR, int D, int WAVES, int UTW, int TR, int esize) {
  if (esize == 2) return GR == 4 && D == 1024 && WAVES == 4 && UTW == 1 ? 2 : 1;
  return esize == 4 && TR == 4 && GR >= 3 && WAVES == 4 && UTW == 1 && D >= 384 ? (D > 512 ? 4 : 2) : 1;
}
constexpr bool fwd_form_4x4x1(int GR, int D, int WAVES, int UTW, int TR, int esize) {
  return esize == 4 && TR == 4 && GR >= 3 && WAVES <= 4 && UTW * D / fwd_k_split(GR, D, WAVES, UTW, TR, esize) <= 384;
}
// (16-bit kernels whose waves split k: the whole operand in registers)
constexpr bool fwd_k_split16(int GR, int D, int WAVES, int UTW, int TR, int esize) {
  return esize == 2 && fwd_k_split(GR, D, WAVES, UTW, TR, esize) > 1;
}
// Forward kernel: one more wave per workgroup that fetches Wx for the compute waves.  A vector memory instruction that a
// compute wave issues behind the exchange wait delays its MFMAs (~70 cycles each on the chain of dependent steps), one
// issued in front of the wait delays the probe (a wave's memory operations return in order).  The producer wave has a
// queue of its own: it loads the Wx of the whole workgroup three steps ahead and writes the Wx of the next step into an
// LDS buffer, from which the compute waves take their elements with LDS reads.  For the kernels with steps of ~2000 cycles
// (16-bit types, 4- and 8-row tiles, heads of several workgroups of 4 waves) that stay within the 256 registers a wave has when
// five share four SIMDs (heads of one workgroup of up to 8 waves, where every load is on the chain: the gated cells,
// GRU B16 T2048 N4 D128 forward 0.915 -> 0.826 ms), and for the cells with four gates: LSTM D = 256 forward 0.944 -> 0.887 ms per 1024 steps, sLSTM
// D = 192 0.961 -> 0.914; the GRU (three loads per step to save) measured +1.5 % to -0.8 %, Elman the same to 0.3 %.
constexpr bool fwd_producer_wave(int GR, int D, int WAVES, int UTW, int KW, int TR, int esize) {
  // (heads of one workgroup: every load is on the chain; the Elman cell, one load per step, measured 0 to +10 % with the wave)
  if (KW == 1) return esize == 2 && GR >= 3 && TR == 4 && WAVES <= 8 && UTW == 1;
  return esize == 2 && GR == 4 && KW > 1 && TR <= 8 && WAVES == 4 && UTW * GR * (D / 32) * 4 <= (TR == 4 ? 160 : 128);
}
// Forward kernel: may the producer wave also store the outputs of a step (16-byte pieces, one step late) instead of the
// compute lanes (2 bytes per state and lane at 4-row tiles)?  Exists for the heads that run as one workgroup with a
// producer wave; the host picks these instantiations for launches that fill the device (measured: LSTM B256 N12 D64
// forward -20 %, but +5-9 % at B = 16, where the stores of the compute lanes are hidden anyway).
constexpr bool fwd_producer_stores(int GR, int D, int WAVES, int UTW, int KW, int TR, int esize) {
  return KW == 1 && fwd_producer_wave(GR, D, WAVES, UTW, KW, TR, esize);
}
// Backward kernel: the same producer wave for the operands of a step (gate cache, s_(t-1), the cotangent of the
// states), for the heads that run as one workgroup: there every load of the compute waves is on the chain of dependent
// steps, and a step (~1600 cycles) is shorter than a fetch from HBM, which their one-step prefetch therefore waits for
// (a timing-only build without these loads runs GRU D = 128 backward 35 % faster).  The producer wave loads four steps
// ahead and leaves the operands of the next step in LDS.  Not in recompute mode, and not for truncated backpropagation
// (no barrier per step to hand over at: that variant of the step keeps its own loads).  All four cells: GRU B16 T2048
// N4 D128 1.396 -> 1.049 ms, Elman B16 T1024 N12 D64 0.312 -> 0.261, N6 D128 0.386 -> 0.301.
constexpr bool bwd_producer_wave(int GR, int nc, int D, int WAVES, int UTW, int KW, int TR, int esize, bool rc) {
  // (nc = 5, the sLSTM: its 8-wave kernel spills at the 170 registers that nine waves leave each)
  return esize == 2 && !rc && KW == 1 && TR == 4 && (WAVES <= 6 || (WAVES <= 8 && nc <= 4)) && UTW == 1;
}
// LDS bytes of the hand-over buffers of that wave (two steps): the gate cache (nc values per element, padded to an even
// number), s_(t-1) and the cotangent (s states each) of the workgroup's UT_WG tiles of TR rows x 16 units, and 16
// spare bytes
constexpr int bwd_producer_bytes(int nc, int s, int ut_wg, int TR, int esize) {
  return 2 * ut_wg * TR * 16 * ((nc + 1) / 2 * 2 + 2 * s) * esize + 16;
}
// Backward kernel: may the producer wave also store dWx (see fwd_producer_stores)?  Not the 8-wave kernels (D = 128): one
// workgroup of nine waves per compute unit is all that their 166 registers allow, and there the variant measured slower
// (LSTM bf16 B256 T1024 N6 D128 reverse kernel 1.46 -> 1.58 ms, GRU 1.18 -> 1.21).
constexpr bool bwd_producer_stores(int GR, int nc, int D, int WAVES, int UTW, int KW, int TR, int esize, bool rc) {
  return bwd_producer_wave(GR, nc, D, WAVES, UTW, KW, TR, esize, rc) && WAVES <= 6;
}
// Backward kernel, fp32 4x4x1 form, gated cells at heads from 384 units on: the four waves of a workgroup pair up over two
// tile positions, and each wave of a pair keeps R^T (own gate rows x destinations) for every second group of 4
// destination workgroups (G_r * D / 8 registers instead of G_r * D / 4) and sends those groups' partial sums itself;
// the first wave of a pair alone owns the pair's elements (gate math, loads, stores, receive).  D = 16 * (WAVES / 2) * KW.
// The same for the 16-bit kernels of the 4-gate cells at D = 1024 (16x16x32 form, every tile height): each wave of a
// pair keeps the fragments of one half of the 32 destination workgroups, 256 registers, none of them in LDS.
// fp32 heads beyond 512 units: one tile position, every fourth group of 4 destinations per wave (G_r * D / 16 registers).
constexpr int bwd_dest_split(int GR, int D, int WAVES, int UTW, int KW, int TR, int esize, bool rc) {
  if (esize == 2) return !rc && GR == 4 && D == 1024 && WAVES == 4 && UTW == 1 && KW == 32 ? 2 : 1;
  return esize == 4 && TR == 4 && !rc && GR >= 3 && WAVES == 4 && UTW == 1 && D >= 384 && KW >= 8 ? (D > 512 ? 4 : 2) : 1;
}
// Backward kernel: LDS bytes of the two dWx hand-over buffers of the producer-store instantiations
// ([gate][row][unit], and [row][unit] for the GRU's g-gate cotangent), behind the operand hand-over buffers
constexpr int bwd_producer_store_bytes(int gw, bool gru, int D, int TR, int esize) {
  return 2 * (gw * TR * (D + 8) + (gru ? TR * (D + 8) : 0)) * esize;
}
// Forward kernel: do the k-steps over the workgroup's own slice of h run in front of the exchange wait?  Heads of
// 2..16 workgroups (up to 12 where part of the operand lives in LDS) whose slice is a whole number of k-steps; not the fp32
// kernels whose operand alone takes 256 registers, at the tile heights where they keep 2 or 4 elements per lane
// (with the two-part product they spill).  The host reads this for the delay of the first probe.
constexpr bool fwd_own_slice_first(int GR, int D, int WAVES, int UTW, int KW, int TR, int esize) {
  const int KM = esize == 4 ? 4 : 32, KS = D / KM;
  return KW > 1 && KW <= 16 && !fwd_form_4x4x1(GR, D, WAVES, UTW, TR, esize) && !fwd_k_split16(GR, D, WAVES, UTW, TR, esize) &&
         (fwd_lds_ksteps(GR, D, WAVES, UTW, esize) == 0 || KW <= 12) && (D / KW) % KM == 0 &&
         !(esize == 4 && UTW * GR * KS >= 256 && TR >= (KW > 8 ? 8 : 16));
}
}

// Measured on MI355X (T = 1024, bf16): when the head fits one workgroup, one tile per wave and
// 8..16 waves (2..4 per SIMD, so one wave's gate math hides behind another's MFMAs) beats 4 waves
// with several tiles each; when it does not fit, 4 waves with one tile each and more workgroups
// beat fewer, fuller workgroups (the step is a dependency chain, not a throughput problem).
// ---- 4 recurrent gate rows per unit (lstm, slstm) --------------------------------------------
// (D = 1024, forward and backward: workgroups of two wave pairs, see fwd_k_split / bwd_dest_split; the reverse kernels
// stop at 8-row tiles: at 16 rows the sLSTM's, with four states, and the fp16 LSTM's spill, and the bf16 LSTM's, which
// does not, takes twice as long per launch as at 8 rows: LSTM bf16 B256 T512 12.5 against 12.8 ms)
#define FRNN_PLANS_GR4_BF16(X) \
  X(32, 0, 2, 1, 1, 16) X(64, 0, 4, 1, 1, 16) X(96, 0, 6, 1, 1, 16) X(128, 0, 8, 1, 1, 16) X(160, 0, 10, 1, 1, 8) X(192, 0, 12, 1, 1, 4) \
  X(256, 0, 4, 1, 4, 16) X(320, 0, 4, 1, 5, 16) X(384, 0, 4, 1, 6, 16) X(448, 0, 4, 1, 7, 16) X(512, 0, 4, 1, 8, 16) X(640, 0, 4, 1, 10, 16) X(768, 0, 4, 1, 12, 8) X(1024, 0, 4, 1, 32, 16)
#define FRNN_BWD_PLANS_GR4_BF16(X) \
  X(160, 2, 2, 1, 5, 16) \
  X(32, 0, 2, 1, 1, 16) X(64, 0, 4, 1, 1, 16) X(96, 0, 6, 1, 1, 16) X(128, 0, 8, 1, 1, 16) X(160, 0, 10, 1, 1, 4) X(192, 0, 4, 1, 3, 16) \
  X(256, 0, 4, 1, 4, 16) X(320, 0, 4, 1, 5, 16) X(384, 0, 4, 1, 6, 16) X(448, 0, 4, 1, 7, 16) X(512, 0, 4, 1, 8, 16) X(640, 0, 4, 1, 10, 16) X(768, 0, 4, 1, 12, 8) X(1024, 0, 4, 1, 32, 8)
// slstm backward: as above, but D = 160 as 5 workgroups of 2 waves (10 waves of 168 registers each spill at every tile height)
#define FRNN_BWD_PLANS_SLSTM_BF16(X) \
  X(128, 2, 4, 1, 2, 16) \
  X(32, 0, 2, 1, 1, 16) X(64, 0, 4, 1, 1, 16) X(96, 0, 6, 1, 1, 8) X(128, 0, 8, 1, 1, 8) X(160, 0, 2, 1, 5, 16) X(192, 0, 4, 1, 3, 16) \
  X(256, 0, 4, 1, 4, 16) X(320, 0, 4, 1, 5, 16) X(384, 0, 4, 1, 6, 16) X(448, 0, 4, 1, 7, 16) X(512, 0, 4, 1, 8, 16) X(640, 0, 4, 1, 10, 16) X(768, 0, 4, 1, 12, 8) X(1024, 0, 4, 1, 32, 8)
// slstm: its heavier gate math tips D = 192 forward to 3 workgroups of 4 waves (1.19 against 1.26 ms)
#define FRNN_PLANS_SLSTM_BF16(X) \
  X(160, 2, 2, 1, 5, 16) \
  X(32, 0, 2, 1, 1, 16) X(64, 0, 4, 1, 1, 16) X(96, 0, 6, 1, 1, 16) X(128, 0, 8, 1, 1, 16) X(160, 0, 10, 1, 1, 8) X(192, 0, 4, 1, 3, 16) \
  X(256, 0, 4, 1, 4, 16) X(320, 0, 4, 1, 5, 16) X(384, 0, 4, 1, 6, 16) X(448, 0, 4, 1, 7, 16) X(512, 0, 4, 1, 8, 16) X(640, 0, 4, 1, 10, 16) X(768, 0, 4, 1, 12, 8) X(1024, 0, 4, 1, 32, 16)
// fp32: a 16-unit tile of a gated cell takes G_r * D / 4 registers of a wave (D in the 4x4x1 form of the 4-row tiles).
// Forward, D = 384 .. 512: workgroups of two wave pairs, 4-row tiles only (see fwd_k_split; D = 16 * (WAVES / 2) * KW);
// D = 640 .. 1024: one tile per workgroup, k split over its four waves, groups that span the device (D = 16 * KW)
#define FRNN_PLANS_GR4_F32(X) \
  X(32, 0, 2, 1, 1, 16) X(64, 0, 4, 1, 1, 16) X(96, 0, 6, 1, 1, 16) X(128, 0, 4, 1, 2, 16) X(160, 0, 2, 1, 5, 16) X(192, 0, 4, 1, 3, 16) X(256, 0, 4, 1, 4, 16) \
  X(320, 0, 4, 1, 5, 8) X(384, 0, 4, 1, 12, 4) X(448, 0, 4, 1, 14, 4) X(512, 0, 4, 1, 16, 4) \
  X(640, 0, 4, 1, 40, 4) X(768, 0, 4, 1, 48, 4) X(1024, 0, 4, 1, 64, 4)
// (backward, D = 384 .. 512: workgroups of two wave pairs, D = 640 .. 1024: one tile position per workgroup, 4-row tiles
// only; see bwd_dest_split)
#define FRNN_BWD_PLANS_GR4_F32(X) \
  X(320, 2, 1, 1, 20, 4) \
  X(64, 2, 2, 1, 2, 16) \
  X(32, 0, 2, 1, 1, 16) X(64, 0, 4, 1, 1, 8) X(96, 0, 2, 1, 3, 16) X(128, 0, 4, 1, 2, 16) X(160, 0, 2, 1, 5, 16) X(192, 0, 4, 1, 3, 16) X(256, 0, 4, 1, 4, 8) \
  X(320, 0, 4, 1, 5, 8) X(384, 0, 4, 1, 12, 4) X(448, 0, 4, 1, 14, 4) X(512, 0, 4, 1, 16, 4) \
  X(640, 0, 4, 1, 40, 4) X(768, 0, 4, 1, 48, 4) X(1024, 0, 4, 1, 64, 4)
// slstm fp32 backward: the same without the 20-workgroup tiling of D = 320 (with four states its kernel spills)
#define FRNN_BWD_PLANS_SLSTM_F32(X) \
  X(64, 2, 2, 1, 2, 16) \
  X(32, 0, 2, 1, 1, 16) X(64, 0, 4, 1, 1, 8) X(96, 0, 2, 1, 3, 16) X(128, 0, 4, 1, 2, 16) X(160, 0, 2, 1, 5, 16) X(192, 0, 4, 1, 3, 16) X(256, 0, 4, 1, 4, 8) \
  X(320, 0, 4, 1, 5, 8) X(384, 0, 4, 1, 12, 4) X(448, 0, 4, 1, 14, 4) X(512, 0, 4, 1, 16, 4) \
  X(640, 0, 4, 1, 40, 4) X(768, 0, 4, 1, 48, 4) X(1024, 0, 4, 1, 64, 4)
// ---- 3 recurrent gate rows per unit (gru) ----------------------------------------------------
#define FRNN_PLANS_GR3_BF16(X) \
  X(32, 0, 2, 1, 1, 16) X(64, 0, 4, 1, 1, 16) X(96, 0, 6, 1, 1, 16) X(128, 0, 8, 1, 1, 16) X(160, 0, 10, 1, 1, 16) X(192, 0, 12, 1, 1, 16) \
  X(256, 0, 4, 1, 4, 16) X(320, 0, 4, 1, 5, 16) X(384, 0, 4, 1, 6, 16) X(448, 0, 4, 1, 7, 16) X(512, 0, 4, 1, 8, 16) X(640, 0, 4, 1, 10, 16) X(768, 0, 4, 1, 12, 16) X(1024, 0, 4, 1, 16, 16)
#define FRNN_BWD_PLANS_GR3_BF16(X) \
  X(192, 2, 4, 1, 3, 16) \
  X(32, 0, 2, 1, 1, 16) X(64, 0, 4, 1, 1, 16) X(96, 0, 6, 1, 1, 16) X(128, 0, 8, 1, 1, 16) X(160, 0, 10, 1, 1, 8) X(192, 0, 12, 1, 1, 4) \
  X(256, 0, 4, 1, 4, 16) X(320, 0, 4, 1, 5, 16) X(384, 0, 4, 1, 6, 16) X(448, 0, 4, 1, 7, 16) X(512, 0, 4, 1, 8, 16) X(640, 0, 4, 1, 10, 16) X(768, 0, 4, 1, 12, 8) X(1024, 0, 4, 1, 16, 16)
#define FRNN_PLANS_GR3_F32(X) \
  X(32, 0, 2, 1, 1, 16) X(64, 0, 4, 1, 1, 16) X(96, 0, 6, 1, 1, 16) X(128, 0, 4, 1, 2, 16) X(160, 0, 2, 1, 5, 16) X(192, 0, 4, 1, 3, 16) X(256, 0, 4, 1, 4, 16) \
  X(320, 0, 4, 1, 5, 16) X(384, 0, 4, 1, 12, 4) X(448, 0, 4, 1, 14, 4) X(512, 0, 4, 1, 16, 4) \
  X(640, 0, 4, 1, 40, 4) X(768, 0, 4, 1, 48, 4) X(1024, 0, 4, 1, 64, 4)
#define FRNN_BWD_PLANS_GR3_F32(X) \
  X(64, 2, 2, 1, 2, 16) \
  X(32, 0, 2, 1, 1, 16) X(64, 0, 4, 1, 1, 16) X(96, 0, 2, 1, 3, 16) X(128, 0, 4, 1, 2, 16) X(160, 0, 2, 1, 5, 16) X(192, 0, 4, 1, 3, 16) X(256, 0, 4, 1, 4, 16) \
  X(320, 0, 4, 1, 5, 16) X(384, 0, 4, 1, 12, 4) X(448, 0, 4, 1, 14, 4) X(512, 0, 4, 1, 16, 4) \
  X(640, 0, 4, 1, 40, 4) X(768, 0, 4, 1, 48, 4) X(1024, 0, 4, 1, 64, 4)
// ---- 1 recurrent gate row per unit (elman) ---------------------------------------------------
#define FRNN_PLANS_GR1_BF16(X) \
  X(32, 0, 2, 1, 1, 16) X(64, 0, 4, 1, 1, 16) X(96, 0, 6, 1, 1, 16) X(128, 0, 8, 1, 1, 16) X(160, 0, 10, 1, 1, 16) X(192, 0, 12, 1, 1, 16) \
  X(256, 0, 16, 1, 1, 16) X(320, 0, 4, 1, 5, 16) X(384, 0, 8, 3, 1, 4) X(448, 0, 4, 1, 7, 16) X(512, 0, 4, 1, 8, 16) X(640, 0, 4, 1, 10, 16) \
  X(768, 0, 8, 1, 6, 16) X(1024, 0, 8, 1, 8, 8)
#define FRNN_BWD_PLANS_GR1_BF16(X) \
  X(32, 0, 2, 1, 1, 16) X(64, 0, 4, 1, 1, 16) X(96, 0, 6, 1, 1, 16) X(128, 0, 8, 1, 1, 16) X(160, 0, 10, 1, 1, 16) X(192, 0, 12, 1, 1, 16) \
  X(256, 0, 16, 1, 1, 16) X(320, 0, 4, 1, 5, 16) X(384, 0, 8, 1, 3, 16) X(448, 0, 4, 1, 7, 16) X(512, 0, 8, 1, 4, 16) X(640, 0, 4, 1, 10, 16) \
  X(768, 0, 8, 1, 6, 16) X(1024, 0, 8, 1, 8, 4)
// (fp32: a 16-unit tile costs D / 4 MFMAs of 32 cycles per step whatever the batch tile, so heads from D = 128 on are
// spread over D / 64 workgroups with one tile per wave: D = 256 as one workgroup of 4 waves x 4 tiles took 8.0 ms
// per 1024 steps forward + backward, as 4 workgroups it takes 2.7)
#define FRNN_PLANS_GR1_F32(X) \
  X(96, 2, 2, 1, 3, 16) \
  X(32, 0, 2, 1, 1, 16) X(64, 0, 4, 1, 1, 16) X(96, 0, 6, 1, 1, 16) X(128, 0, 4, 1, 2, 16) X(160, 0, 2, 1, 5, 16) X(192, 0, 4, 1, 3, 16) X(256, 0, 4, 1, 4, 16) \
  X(320, 0, 4, 1, 5, 16) X(384, 0, 4, 1, 6, 16) X(448, 0, 4, 1, 7, 16) X(512, 0, 4, 1, 8, 16) X(640, 0, 4, 1, 10, 16) X(768, 0, 4, 1, 12, 8) X(1024, 0, 4, 1, 16, 8)
#define FRNN_BWD_PLANS_GR1_F32(X) \
  X(96, 2, 2, 1, 3, 16) \
  X(32, 0, 2, 1, 1, 16) X(64, 0, 4, 1, 1, 16) X(96, 0, 6, 1, 1, 16) X(128, 0, 4, 1, 2, 16) X(160, 0, 2, 1, 5, 16) X(192, 0, 4, 1, 3, 16) X(256, 0, 4, 1, 4, 16) \
  X(320, 0, 4, 1, 5, 16) X(384, 0, 4, 1, 6, 16) X(448, 0, 4, 1, 7, 16) X(512, 0, 4, 1, 8, 16) X(640, 0, 4, 1, 10, 16) X(768, 0, 4, 1, 12, 16) X(1024, 0, 4, 1, 16, 8)

// ---- reverse scan in recompute mode (no gate cache): R and R^T are both resident, so only the head
// dims whose two operands fit the registers beside the working set; same tilings as above where those
// fit (gru D = 192 runs as 3 workgroups of 4 waves here: 12 waves have 168 registers each).  D = 320 (and 384 for the
// GRU, three gate rows) at 4-row tiles only; the 4-gate cells spill at D = 384, the GRU at D = 512.
#define FRNN_BWD_RC_PLANS_GR4_BF16(X) \
  X(32, 0, 2, 1, 1, 16) X(64, 0, 4, 1, 1, 16) X(96, 0, 6, 1, 1, 4) X(128, 0, 4, 1, 2, 16) X(192, 0, 4, 1, 3, 16) X(256, 0, 4, 1, 4, 8) X(320, 0, 4, 1, 5, 4)
// slstm: D = 192 stops at 8-row tiles (its 16-row kernel, with both operands resident and four states, spills)
#define FRNN_BWD_RC_PLANS_SLSTM_BF16(X) \
  X(32, 0, 2, 1, 1, 16) X(64, 0, 4, 1, 1, 16) X(96, 0, 6, 1, 1, 4) X(128, 0, 4, 1, 2, 16) X(192, 0, 4, 1, 3, 8) X(256, 0, 4, 1, 4, 8) X(320, 0, 4, 1, 5, 4)
#define FRNN_BWD_RC_PLANS_GR3_BF16(X) \
  X(32, 0, 2, 1, 1, 16) X(64, 0, 4, 1, 1, 16) X(96, 0, 6, 1, 1, 8) X(128, 0, 8, 1, 1, 8) X(192, 0, 4, 1, 3, 16) X(256, 0, 4, 1, 4, 16) X(320, 0, 4, 1, 5, 4) X(384, 0, 4, 1, 6, 4)
#define FRNN_BWD_RC_PLANS_GR4_F32(X) X(32, 0, 2, 1, 1, 16) X(64, 0, 4, 1, 1, 16)
#define FRNN_BWD_RC_PLANS_GR3_F32(X) X(32, 0, 2, 1, 1, 16) X(64, 0, 4, 1, 1, 16)
#define FRNN_BWD_RC_PLANS_NONE(X)
