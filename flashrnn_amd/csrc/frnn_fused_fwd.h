// Fused forward: one persistent kernel runs all T steps.
//
// Replaces FLASHRNNCellFusedForward, flashrnn/flashrnn/fused/flashrnn_fused_forward.cu:146-659.
//
// Work split.  A "unit tile" is 16 hidden units of one head with all their G_r gate rows.
// A wave owns UTW unit tiles and keeps their R rows (all K = D columns) in registers as MFMA
// A operands for the whole sequence.  A workgroup has WAVES waves; KW workgroups share one
// (head, 16-row batch tile) group: D = 16 * UTW * WAVES * KW.  Groups are independent.
//
// One step:  h_{t-1} (16 x D, storage type) sits in LDS in fragment order
//   -> per k-step one LDS read per lane, G_r*UTW MFMAs (A = R rows, B = h^T, fp32 acc)
//   -> lane (col b = lane%16, rows 4*(lane/16)..+3) holds every gate of 4 units of batch row b
//   -> gates, new states in fp32 registers; states / gate cache stored straight in the public
//      / private layouts; the new h goes to the other LDS buffer (KW == 1) or to the tagged
//      global exchange (KW > 1).
// Nothing inside a step branches on the lane: padded batch rows are handled by out-of-range
// buffer offsets, so the compiler can count outstanding memory operations exactly and the Wx
// prefetch and the output stores never stall the recurrence.  The bias is the C operand of the
// first MFMA of each gate.
#pragma once
#include "frnn_exchange.h"
#include "frnn_mailbox.h"
#include "frnn_plan.h"
#include "frnn_pointwise.h"

namespace frnn {

struct FwdArgs {
  const void* Wx; const void* R; const void* b; const void* s0;
  void* states; void* cache;
  u64* ll; int* status;
  int* xcd;          // 32 words per group for xcd_handshake (zero at launch), or null: exchange stores stay agent scope
  int B, T, N;
  int BS;  // rows between the state planes of s0 and states ([S, BS, ...]); B unless the call covers a range of a larger batch
  int grp0, groups, groups_total;  // this launch handles groups [grp0, grp0 + groups)
  int tile_rows;                   // batch rows per group: 4, 8 or 16
  int training, spin_limit, poll_delay;
  // single-step calls (T == 1, state carried from call to call): `carry` [S][B][N][D] fp32, if not null,
  // holds the unrounded state: it is read instead of s0 for the gate math and rewritten at the end, so that
  // a sequence of steps computes bit for bit what one call over the sequence does (which carries the state in
  // fp32 registers); h for the recurrent product still comes from s0, in the storage type, as in the time loop.
  // step != 0: all groups send their (unread) exchange words to one area
  float* carry; int step;
  float h_clip;      // > 0: new h clamped to [-h_clip, h_clip] (forward_clipval)
  int pst;           // host side only: launch the instantiation whose producer wave stores the outputs (fwd_producer_stores)
  // resident decode kernel (the MB instantiations): T = the most tokens the launch serves; the Wx of token t is taken
  // from the inbox of `mailbox` and the new states go to its outbox (frnn_mailbox.h); a wait for a token gives up after
  // idle_limit probes or when the stop word of the control block is set, and the kernel then ends normally
  void* mailbox; size_t inbox_off, outbox_off, in_slot, out_slot; int slots, idle_limit;
  long long* trace;  // phase cycle sums per workgroup; only written by -DFRNN_TRACE builds
};

#ifdef FRNN_TRACE
#define FRNN_STAMP(var) __builtin_amdgcn_sched_barrier(0); const long long var = clock64(); __builtin_amdgcn_sched_barrier(0)
#else
#define FRNN_STAMP(var)
#endif

template <typename T> __device__ __forceinline__ typename ST<T>::Frag load_frag(const T* row, int ks, int kq);
template <> __device__ __forceinline__ bf16x8 load_frag<bf16_t>(const bf16_t* row, int ks, int kq) {
  return *reinterpret_cast<const bf16x8*>(row + ks * 32 + kq * 8);
}
template <> __device__ __forceinline__ f16x8 load_frag<half_t>(const half_t* row, int ks, int kq) {
  return *reinterpret_cast<const f16x8*>(row + ks * 32 + kq * 8);
}
template <> __device__ __forceinline__ float load_frag<float>(const float* row, int ks, int kq) {
  return row[ks * 4 + kq];
}

template <int F, typename T, int D, int WAVES, int UTW, int KW, int TR, bool MB = false, bool PSTV = false>
__global__ void __launch_bounds__((WAVES + (!MB && fwd_producer_wave(Cell<F>::GR, D, WAVES, UTW, KW, TR, (int)sizeof(T)) ? 1 : 0)) * 64)
fused_fwd_kernel(const FwdArgs a) {
  static_assert(!MB || TR == 4, "the resident decode kernel runs on 4-row batch tiles");
  typedef Cell<F> C;
  typedef ST<T> X;
  typedef CellMath<F, X::FAST> CM;
  typedef typename X::Vec4 Vec4;
  typedef typename X::Frag Frag;
  typedef Own<TR> O;
  constexpr int GR = C::GR, GW = C::GW, GT = C::GT, S = C::S, NC = C::NC;
  // (KSP = 2: the fp32 4x4x1 form of heads from 384 units on, two waves per tile, each with one half of k; 4 beyond 512 units)
  constexpr int KSP = fwd_k_split(GR, D, WAVES, UTW, TR, (int)sizeof(T)), DK = D / KSP;
  constexpr int KS = D / X::KM, NT = WAVES * 64, UT_WG = WAVES * UTW / KSP;
  static_assert(UT_WG * KW * 16 == D, "tiling must cover the head");
  static_assert(KSP <= 2 || (sizeof(T) == 4 && UTW == 1), "more than two waves per tile: the fp32 4x4x1 form only");
  constexpr int LLW = 16 * D / X::EPW;  // 64-bit words per exchange slot
  // words a thread polls per step: the TR rows of the tile, without the workgroup's own slice
  // (polled 16 at a time: longer lists are padded to whole rounds with entries that wait for nothing)
  constexpr int NP_ = (LLW * TR / 16 * (KW > 1 ? KW - 1 : 1) / KW + NT - 1) / NT;
  // 16-bit types fetch two adjacent words with one 16-byte load when a thread polls more than one
  constexpr bool PAIRS = X::EPW == 2 && NP_ > 1;
  constexpr int NP = NP_ <= 16 ? (PAIRS ? (NP_ + 1) / 2 * 2 : NP_) : (NP_ + 15) / 16 * 16;
  // (values per element of a cache line: the cell's NC and, where cache_carried_state says so, one state of step t-1)
  constexpr int CXS = cache_carried_state(F, (int)sizeof(T), D), NCX = NC + (CXS >= 0 ? 1 : 0);
  constexpr int NCA = NCX > 0 ? NCX : 1;
  constexpr int GX = GT - GR > 0 ? GT - GR : 1;
  constexpr int E = O::E, ND_ = NDW<T, E>::value;
  constexpr bool SB = NDW<T, E>::SUB;  // single bf16 elements: 16-bit memory operations
  constexpr unsigned ES = sizeof(T);

  // fp32, 4-row batch tiles, cells with 3 or 4 recurrent gates: the product runs on v_mfma_f32_4x4x1_16B_f32 with
  // the 4 batch rows on the 4-wide side, so that no MFMA work goes into padded batch columns (the 16x16x4
  // instruction computes 16 columns, 12 of them padding, at the same rate).  Block = unit of the tile, the 4
  // columns of a block = the gates of that unit, A = h (the values of one block broadcast to all 16), one
  // instruction per k: D instructions of 8 cycles per tile and step instead of G_r * D / 4 of 32.
  constexpr bool M44 = fwd_form_4x4x1(GR, D, WAVES, UTW, TR, (int)sizeof(T));  // (the whole operand, D registers per tile, in registers)
  constexpr bool KS16 = fwd_k_split16(GR, D, WAVES, UTW, TR, (int)sizeof(T));  // 16-bit kernels whose wave pairs split k
  constexpr int KSW = KS16 ? KS / KSP : KS;  // k-steps of a wave
  constexpr int RLK = M44 || KS16 ? 0 : fwd_lds_ksteps(GR, D, WAVES, UTW, (int)sizeof(T)), KSR = KSW - RLK;
  // Own slice first: of the h_(t-1) a step multiplies with, the workgroup's own D / KW units are in LDS as soon as
  // its waves have finished step t-1; the k-steps over them run before the wait for the other workgroups' slices
  // (behind one more LDS barrier) and leave the critical path.  Each workgroup keeps R and h rotated along k so
  // that its own slice comes first: k-step ks of the loops below is k-step (ks + slice * KSO) % KS of the head.
#ifdef FRNN_NO_OWN_FIRST
  constexpr bool OWN_FIRST = false;
#else
  constexpr bool OWN_FIRST = fwd_own_slice_first(GR, D, WAVES, UTW, KW, TR, (int)sizeof(T));
#endif
  constexpr int KSO = OWN_FIRST ? (D / KW) / X::KM : 0;
  __shared__ __attribute__((aligned(16))) T hbuf[2][16 * D];
  __shared__ int dead_flag, near_word, stop_flag, stop_reason;
  // Wx of one step for the whole workgroup, two buffers by step parity: [tile][gate][batch row][16 units]
  constexpr bool PW = !MB && fwd_producer_wave(GR, D, WAVES, UTW, KW, TR, (int)sizeof(T));  // (a token's Wx cannot be fetched ahead)
  constexpr int WBUF = UT_WG * GW * TR * 16;
  __shared__ __attribute__((aligned(16))) T wbuf[PW ? 2 * WBUF + 8 : 1];  // (+ 16 bytes that swallow the writes of lanes without a piece)
  // Producer-wave stores (PSTV instantiations of the heads that run as one workgroup with a producer wave; chosen on the
  // host for launches that fill the device, where the kernel is bound by memory traffic): at 4-row tiles a compute
  // lane owns one element and stores 2 bytes per state and step, 9.4 M store instructions per launch at B = 256; here
  // the compute waves leave the step's states and cache values in LDS as they lie in memory, two buffers by step
  // parity, and the producer wave stores them one step later in 16-byte pieces.
  constexpr bool PST = PSTV && PW && KW == 1;
  constexpr int NCP_O = CacheBlk<T, NCA>::NCP;
  // (rows of the state part are D + 8 elements apart: at a stride of 128 bytes, D = 64, rows 0 and 2 of a tile would meet
  // in the same banks under the lanes' 2-byte writes)
  constexpr int OBR = D + 8;
  constexpr int OB_ST = S * TR * OBR, OB_CA = NC > 0 ? UT_WG * TR * 16 * NCP_O : 0, OB = OB_ST + OB_CA;  // [state][row][unit] [tile][row][unit][value]
  __shared__ __attribute__((aligned(16))) T obuf[PST ? 2 * OB : 1];
  // [wave][k-step][u][g][lane]: each lane reads back what it wrote
  __shared__ __attribute__((aligned(16))) Frag rlds[RLK > 0 ? WAVES * RLK * UTW * GR * 64 : 1];
  __shared__ f32x4 psum[KSP > 1 ? UT_WG * (KS16 ? GR : KSP - 1) * 64 : 1];  // partial sums of the other waves of a tile: [tile][(gate | wave)][lane]

  int grp_l, slice;
  if (!decode_block(a.groups, KW, grp_l, slice)) return;
  const int grp = a.grp0 + grp_l;
  const int N = a.N, Tn = a.T, B = a.B, BS = a.BS;
  const int n = grp % N, bt = grp / N;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int r16 = lane & 15, q4 = lane >> 4;
  const int brow = O::row(r16), esub = O::sub(r16, q4);
  const int bg = bt * TR + brow;  // batch row this lane does the gate math for
  // wave w of a pair-split workgroup: tile w / 2 of the workgroup, half w % 2 of k; the lanes of a second-half wave
  // own no element (every load of theirs returns zero, every store is dropped)
  const int kh = KSP > 1 ? w % KSP : 0, wt = KSP > 1 ? w / KSP : w;
  const bool bvalid = bg < B && kh == 0;
  const int rows_valid = min(TR, B - bt * TR);
  const unsigned Bpad = (unsigned)B;  // rows of the gate cache: padded rows are never read or written
  const T* __restrict__ R = static_cast<const T*>(a.R);
  const T* __restrict__ bias_g = static_cast<const T*>(a.b);
  const T* __restrict__ s0 = static_cast<const T*>(a.s0);
  const unsigned ND = (unsigned)N * D;
  if (tid == 0) { dead_flag = 0; stop_flag = 0; stop_reason = MB_END_NONE; }
  // (a head of one workgroup never waits, so nothing else writes its call's status word: the host launches no clearing
  // kernel for such a call and the word is set here)
  if constexpr (KW == 1) { if (blockIdx.x == 0 && tid == 0) *a.status = 0; }

  const rsrc_t rWx = make_rsrc(a.Wx, (size_t)B * Tn * GW * ND * ES);
  const rsrc_t rSt = make_rsrc(a.states, ((size_t)(S - 1) * BS + B) * Tn * ND * ES);
  constexpr int NCP = CacheBlk<T, NCA>::NCP, NWC = CacheBlk<T, NCA>::template Words<E>::value;
  const rsrc_t rCa = make_rsrc(a.cache, (size_t)Tn * N * Bpad * D * (NC ? NCP : 0) * ES);

  // ---- the producer wave (see fwd_producer_wave): the workgroup's last wave.  It takes part in every barrier of the
  //      compute waves, in the same order and under the same conditions (all of them wave-uniform values that every
  //      wave reads from LDS behind a barrier).  Wx of step s travels in register set s % 3; iteration t (the compute
  //      waves are in step t and read buffer t & 1) writes Wx(t+1) into the other buffer, which the compute waves read
  //      behind the barriers of step t+1, and then sends for Wx(t+3) --------------------------------------------------
  if constexpr (PW) {
    if (w == WAVES) {
      constexpr int CH_TOT = UT_WG * GW * TR * 2, NCH = (CH_TOT + 63) / 64;  // 16-byte pieces (8 units) per step, per lane
      unsigned pv[NCH]; int pl[NCH];
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        const int c = lane + 64 * i, half = c & 1, pr = (c >> 1) % TR, pg = ((c >> 1) / TR) % GW, ptile = (c >> 1) / (TR * GW);
        const bool ok = c < CH_TOT && bt * TR + pr < B;
        pv[i] = ok ? ((((unsigned)(bt * TR + pr) * Tn * GW + pg) * ND + n * D + slice * (D / KW) + ptile * 16 + half * 8) * ES) : kInvalidOff;
        pl[i] = c < CH_TOT ? ((ptile * GW + pg) * TR + pr) * 16 + half * 8 : -1;  // (-1: the spare 16 bytes behind the buffers)
      }
      Dw<4> set[3][NCH];
      auto fetch = [&](Dw<4> (&dst)[NCH], int s_) __attribute__((always_inline)) {
        const int sc = s_ < Tn ? s_ : Tn - 1;
#pragma unroll
        for (int i = 0; i < NCH; ++i) dst[i] = buf_load<4>(rWx, pv[i], (unsigned)sc * GW * ND * ES);
      };
      auto put = [&](const Dw<4> (&src)[NCH], int s_) __attribute__((always_inline)) {
        // (no branch on the lane: behind one the compiler waits for every load in flight, the latest ones included)
#pragma unroll
        for (int i = 0; i < NCH; ++i)
          *reinterpret_cast<uint4*>(wbuf + (pl[i] >= 0 ? (s_ & 1) * WBUF + pl[i] : 2 * WBUF)) = make_uint4(src[i].v[0], src[i].v[1], src[i].v[2], src[i].v[3]);
      };
      // producer-wave stores: the 16-byte pieces of a step's outputs that this lane stores (states, then gate cache)
      constexpr int SP_TOT = PST ? S * TR * (D / 8) : 0, NSP = (SP_TOT + 63) / 64;
      constexpr int CPR = NCP_O * 2;  // pieces per (tile, batch row) of the cache
      constexpr int CP_TOT = PST && NC > 0 ? UT_WG * TR * CPR : 0, NCQ = (CP_TOT + 63) / 64;
      unsigned svo[NSP > 0 ? NSP : 1], cvo[NCQ > 0 ? NCQ : 1]; int sl[NSP > 0 ? NSP : 1], cl[NCQ > 0 ? NCQ : 1];
#pragma unroll
      for (int i = 0; i < NSP; ++i) {
        const int c = lane + 64 * i, ch = c % (D / 8), pr = (c / (D / 8)) % TR, pk = c / ((D / 8) * TR);
        const bool ok = c < SP_TOT && bt * TR + pr < B;
        svo[i] = ok ? ((((unsigned)(pk * BS + bt * TR + pr) * Tn) * ND + n * D + ch * 8) * ES) : kInvalidOff;
        sl[i] = c < SP_TOT ? (pk * TR + pr) * OBR + ch * 8 : 0;
      }
#pragma unroll
      for (int i = 0; i < NCQ; ++i) {
        const int c = lane + 64 * i, q = c % CPR, pr = (c / CPR) % TR, ptile = c / (CPR * TR);
        const bool ok = c < CP_TOT && bt * TR + pr < B && a.training;
        cvo[i] = ok ? ((((unsigned)ptile * Bpad + bt * TR + pr) * 16) * NCP_O * ES + q * 16) : kInvalidOff;
        cl[i] = c < CP_TOT ? OB_ST + ((ptile * TR + pr) * 16) * NCP_O + q * 8 : 0;
      }
      auto drain = [&](int s_) __attribute__((always_inline)) {  // the outputs of step s_, complete in obuf[s_ & 1]
        const T* const ob = obuf + (s_ & 1) * OB;
#pragma unroll
        for (int i = 0; i < NSP; ++i) {
          const uint4 v = *reinterpret_cast<const uint4*>(ob + sl[i]);
          buf_store<4>(Dw<4>{{v.x, v.y, v.z, v.w}}, rSt, svo[i], (unsigned)s_ * ND * ES);
        }
#pragma unroll
        for (int i = 0; i < NCQ; ++i) {
          const uint4 v = *reinterpret_cast<const uint4*>(ob + cl[i]);
          buf_store<4>(Dw<4>{{v.x, v.y, v.z, v.w}}, rCa, cvo[i], (((unsigned)s_ * N + n) * (D / 16)) * Bpad * 16 * NCP_O * ES);
        }
      };
      fetch(set[0], 0); fetch(set[1], 1); fetch(set[2], 2);
      put(set[0], 0);
      __syncthreads();  // (the one of the prologue below)
      bool pdead = KW > 1 && __builtin_amdgcn_readfirstlane(near_word) < 0;
      auto iter = [&](int t, const Dw<4> (&next)[NCH], Dw<4> (&refill)[NCH]) __attribute__((always_inline)) {
        if (t > 0) {
          if constexpr (OWN_FIRST) lds_barrier();
          if constexpr (KW > 1) { if (barrier_or(false, &dead_flag)) { pdead = true; return; } }
          else lds_barrier();
        }
        put(next, t + 1);
#ifdef FRNN_PST_DRAIN_FIRST
        if constexpr (PST) { if (t > 0) drain(t - 1); }
        fetch(refill, t + 3);
#else
        // (loads before stores: a wave's memory operations complete in order, and a store is acknowledged late when the
        // device is writing at its limit; issued in front of them, the loads that the hand-over two steps on waits for
        // only have stores of an earlier step ahead of them)
        fetch(refill, t + 3);
        if constexpr (PST) { if (t > 0) drain(t - 1); }
#endif
      };
      int t = 0;
      for (; t + 2 < Tn && !pdead; t += 3) {
        iter(t, set[1], set[0]);
        if (pdead) break;
        iter(t + 1, set[2], set[1]);
        if (pdead) break;
        iter(t + 2, set[0], set[2]);
      }
      if (!pdead && t < Tn) {
        iter(t, set[1], set[0]);
        if (!pdead && t + 1 < Tn) iter(t + 1, set[2], set[1]);
      }
      if constexpr (PST) {  // the last step's outputs, behind the barrier that follows the time loop
        lds_barrier();
        drain(Tn - 1);
      }
      return;
    }
  }

  // mailbox records of this lane's elements (resident decode kernel): one inbox and one outbox record per tile
  typedef MbRec<T, GW> RI;
  typedef MbRec<T, S> RO;
  int* const mb_ctrl = static_cast<int*>(a.mailbox);
  const rsrc_t rIn = make_rsrc(MB ? static_cast<char*>(a.mailbox) + a.inbox_off : nullptr, MB ? (size_t)a.slots * a.in_slot : 0);
  const rsrc_t rOut = make_rsrc(MB ? static_cast<char*>(a.mailbox) + a.outbox_off : nullptr, MB ? (size_t)a.slots * a.out_slot : 0);
  unsigned mi_v[MB ? UTW : 1], mo_v[MB ? UTW : 1];
  int ub[UTW];
  unsigned wx_v[UTW], st_v[UTW], ca_v[UTW];  // per-lane byte offsets; out of range for padded rows
#pragma unroll
  for (int u = 0; u < UTW; ++u) {
    ub[u] = (slice * UT_WG + wt * UTW + u) * 16;
    const unsigned d0 = n * D + ub[u] + esub;
    if constexpr (MB) {
      mi_v[u] = bvalid ? ((unsigned)bg * ND + d0) * RI::BYTES : kInvalidOff;
      mo_v[u] = bvalid ? ((unsigned)bg * ND + d0) * RO::BYTES : kInvalidOff;
    }
    wx_v[u] = bvalid ? ((unsigned)bg * Tn * GW * ND + d0) * ES : kInvalidOff;
    st_v[u] = bvalid ? ((unsigned)bg * Tn * ND + d0) * ES : kInvalidOff;
    ca_v[u] = (bvalid && a.training) ? ((((unsigned)(ub[u] >> 4) * Bpad + bg) * 16 + (esub & 15)) * NCP) * ES : kInvalidOff;
  }

  // ---- resident operands ----------------------------------------------------------------
  constexpr int FRAG_REGS = (int)sizeof(Frag) / 4, RF_REGS = UTW * GR * KSR * FRAG_REGS;
  constexpr int PIN_REGS = RF_REGS > 160 ? (RF_REGS < 232 ? RF_REGS : 232) : 0;  // (160 registers, D = 320: measured no gain)
  Frag rf[UTW][GR][KSR];
  const int rot_ks = OWN_FIRST ? slice * KSO : 0, rot_u = OWN_FIRST ? slice * (D / KW) : 0;  // rotation in k-steps, in units
  Frag* const rl = rlds + (size_t)w * RLK * UTW * GR * 64 + lane;
  // 4x4x1 form: lane 4*blk + j holds row (gate j, unit blk of the tile) of R, one register per k
  float rb[M44 ? UTW : 1][M44 ? DK : 1];
  if constexpr (M44) {
    const int blk = lane >> 2, j = lane & 3;
#pragma unroll
    for (int u = 0; u < UTW; ++u) {
      const float* row = reinterpret_cast<const float*>(R) + ((size_t)((j < GR ? j : 0) * N + n) * D + ub[u] + blk) * D + kh * DK;
#pragma unroll
      for (int k = 0; k < DK; k += 4) {
        const float4 v = *reinterpret_cast<const float4*>(row + k);
        rb[u][k] = j < GR ? v.x : 0.f; rb[u][k + 1] = j < GR ? v.y : 0.f;
        rb[u][k + 2] = j < GR ? v.z : 0.f; rb[u][k + 3] = j < GR ? v.w : 0.f;
      }
#ifndef FRNN_NO_AGPR_PIN
      // (as for the fragments below: what does not fit the architectural VGPRs beside the working set is pinned to
      // accumulation registers, where the MFMA reads it in place, instead of being copied back before every use)
      constexpr int PIN44 = UTW * DK - 128 > 232 ? 232 : UTW * DK - 128;
#pragma unroll
      for (int k = 0; k < DK; ++k)
        if (u * DK + (DK - 1 - k) < PIN44) asm volatile("" : "+a"(rb[u][k]));
#endif
    }
  }
#pragma unroll
  for (int u = 0; u < (M44 ? 0 : UTW); ++u)
#pragma unroll
    for (int g = 0; g < GR; ++g) {
      const T* row = R + ((size_t)(g * N + n) * D + ub[u] + r16) * D;
#pragma unroll
      for (int ks = 0; ks < KSW; ++ks) {
        // k-step of the head (own slice first: rotated; wave pairs that split k: this wave's half)
        const int kstep = OWN_FIRST ? (ks + rot_ks < KS ? ks + rot_ks : ks + rot_ks - KS) : KS16 ? kh * KSW + ks : ks;
        const Frag f = load_frag<T>(row, kstep, q4);
        if (ks < KSR) {
          rf[u][g][ks < KSR ? ks : 0] = f;
#ifndef FRNN_NO_AGPR_PIN
          // A resident operand of more than 128 registers does not fit the 256 architectural VGPRs beside the
          // working set.  Left to the register allocator, some fragments are spilled to accumulation registers
          // and copied back (4 moves) in front of every MFMA that uses them; pinned there from the start, the
          // MFMA reads them in place.  As many as the 256 accumulation registers hold, last k-steps first.
          if constexpr (PIN_REGS > 0) {
            if (((u * GR + g) * KSR + (KSR - 1 - ks)) * FRAG_REGS + FRAG_REGS <= PIN_REGS) asm volatile("" : "+a"(rf[u][g][ks]));
          }
#endif
        }
        else rl[(((ks - KSR) * UTW + u) * GR + g) * 64] = f;
      }
    }
  // bias of the recurrent gate slots: as the C operand of the first MFMA when a lane keeps all 4
  // elements of a tile (costs nothing), else added to the lane's own elements in the gate math
  // (4 registers per gate and tile would hold values the lane never uses)
  constexpr bool BIAS_C = E == 4;
  f32x4 biasc[BIAS_C ? UTW : 1][GR];
  float bown[UTW][GR][BIAS_C ? 1 : E];
  float bx[UTW][E][GX];   // bias of the gate slots without recurrent input
  float s[UTW][E][S];
#pragma unroll
  for (int u = 0; u < UTW; ++u) {
#pragma unroll
    for (int g = 0; g < GR; ++g) {
      if constexpr (BIAS_C) {
        float v[4];
        unpack4<T>(*reinterpret_cast<const Vec4*>(bias_g + (size_t)(g * N + n) * D + ub[u] + q4 * 4), v);
        biasc[u][g] = kh == 0 ? f32x4{v[0], v[1], v[2], v[3]} : f32x4{0.f, 0.f, 0.f, 0.f};  // (once per pair of waves)
      } else {
#pragma unroll
        for (int e = 0; e < E; ++e) bown[u][g][e] = (float)bias_g[(size_t)(g * N + n) * D + ub[u] + esub + e];
      }
    }
#pragma unroll
    for (int e = 0; e < E; ++e) {
#pragma unroll
      for (int g = GR; g < GT; ++g) bx[u][e][g - GR] = (float)bias_g[(size_t)(g * N + n) * D + ub[u] + esub + e];
#pragma unroll
      for (int k = 0; k < S; ++k)
        s[u][e][k] = !bvalid ? 0.f : a.carry ? a.carry[((size_t)k * B + bg) * ND + (size_t)n * D + ub[u] + esub + e]
                                              : (float)s0[((size_t)k * BS + bg) * ND + (size_t)n * D + ub[u] + esub + e];
    }
  }

  // ---- h_0 of the whole head -> LDS (rows beyond B are zero and stay zero or private to their
  //      own MFMA column, so they never reach a valid row) --------------------------------------
  for (int idx = tid; idx < (M44 ? 4 : 16) * D / 4; idx += NT) {
    const int row = idx / (D / 4), k0 = (idx % (D / 4)) * 4;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    const bool rv = row < TR && bt * TR + row < B;
    if (rv) unpack4<T>(*reinterpret_cast<const Vec4*>(s0 + (size_t)(bt * TR + row) * ND + (size_t)n * D + k0), v);
    if constexpr (M44) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        reinterpret_cast<float*>(hbuf[0])[lds_index4(row, k0 + i)] = v[i];
        if (!rv) reinterpret_cast<float*>(hbuf[1])[lds_index4(row, k0 + i)] = v[i];
      }
    } else {
      const int kl = OWN_FIRST ? (k0 >= rot_u ? k0 - rot_u : k0 - rot_u + D) : k0;
      lds_write<4>(hbuf[0], row, kl, v);
      if (KW > 1 || TR < 16) {  // rows that are never rewritten must be finite in both buffers
        if (!rv) lds_write<4>(hbuf[1], row, kl, v);
      }
    }
  }

  int qpoll[NP];
  if (KW > 1) ll_plan<T, NP, NT, PAIRS>(tid, rows_valid, D, slice * (D / KW), D / KW, qpoll);
  // per group: slot 0, slot 1, and a third area that swallows the stores of padded lanes
  u64* const llbase = a.ll + (size_t)(a.step ? 0 : grp) * 3 * LLW;
  const rsrc_t rLL = make_rsrc(llbase, (size_t)2 * LLW * 8);  // the two slots that are read
  const int rot_w = rot_u * 16 / X::EPW;  // the rotation in words of the LDS vector (an exchange word holds 32 bits of it)

  // Wx is fetched PD steps ahead into a ring of PD + 1 register sets.  A head that exchanges
  // nothing (KW = 1) has steps shorter than a fetch from HBM takes (D = 64: 1100 cycles against
  // ~1900), so it looks further ahead and issues the loads behind its MFMAs; with an exchange the
  // loads must stay well clear of the poll, whose wait counts every load in flight.
#ifdef FRNN_PD
  constexpr int PD = KW == 1 ? FRNN_PD : 1;
#else
  constexpr int PD = KW > 1 || WAVES >= 16 ? 1 : (D <= 64 ? 3 : 2);  // measured; 16 waves have no registers to spare
#endif
  constexpr bool WX_LATE = KW == 1;
  Dw<ND_> wx[PD + 1][UTW][GW];
  auto load_wx = [&](Dw<ND_> (&dst)[UTW][GW], int t) __attribute__((always_inline)) {
    if constexpr (PW || MB) return;  // (the producer wave's job; the mailbox's)
#pragma unroll
    for (int u = 0; u < UTW; ++u)
#pragma unroll
      for (int g = 0; g < GW; ++g) dst[u][g] = buf_load<ND_, SB>(rWx, wx_v[u], ((unsigned)t * GW + g) * ND * ES);
  };
#pragma unroll
  for (int i = 0; i < PD; ++i) load_wx(wx[i], min(i, Tn - 1));
  // exchange stores may stay in the L2 of the XCD once the group is known to share one (a single step sends
  // nothing that is read)
  if (KW > 1 && w == 0) {
    const int r = (a.xcd && Tn > 1 && !a.step) ? xcd_handshake<KW>(a.xcd + (size_t)grp * 32, slice, lane, a.status, a.spin_limit) : 0;
    if (lane == 0) near_word = r;
  }
  __syncthreads();
  const int near_i = KW > 1 ? __builtin_amdgcn_readfirstlane(near_word) : 0;  // 1: stores stay in the XCD's L2, -1: wait ran out
  u64 near_m;  // lane mask for ll_store_sel: all ones or zero, in scalar registers
  asm("s_cmp_gt_i32 %1, 0\n\ts_cselect_b64 %0, -1, 0" : "=s"(near_m) : "s"(near_i) : "scc");

#ifdef FRNN_TRACE
  long long tr[3] = {0, 0, 0};
  const long long tr_begin = clock64();
#endif
  bool dead = near_i < 0;
  bool stopped = false;  // resident decode kernel: a wait for a token gave up (idle bound or stop word)
  // one time step: consumes `wc` (Wx of step t), prefetches Wx of step t+PD into `wn`
  auto step = [&](const int t, Dw<ND_> (&wc)[UTW][GW], Dw<ND_> (&wn)[UTW][GW]) __attribute__((always_inline)) {
    const int cur = t & 1;
    FRNN_STAMP(c0);
    // NACC accumulators per (tile, gate), used round robin over the k-steps, so that at least ~4
    // independent MFMA chains are in flight (a dependent MFMA waits ~3x longer than an independent one)
    constexpr int NACC_ = UTW * GR >= 3 ? 1 : (UTW * GR == 2 ? 2 : 4);
    constexpr int NACC = NACC_ < KS ? NACC_ : KS;
    f32x4 accp[M44 ? 1 : NACC][UTW][GR];
    if constexpr (OWN_FIRST) {
      if (t > 0) lds_barrier();  // the own slice of h_(t-1), written by the gate math of every wave
      const Frag* hf = reinterpret_cast<const Frag*>(hbuf[cur]) + lane;
      Frag ho[KSO];
#pragma unroll
      for (int k = 0; k < KSO; ++k) ho[k] = hf[k * 64];
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int k = 0; k < KSO; ++k) {
#pragma unroll
        for (int u = 0; u < UTW; ++u)
#pragma unroll
          for (int g = 0; g < GR; ++g)
            accp[k % NACC][u][g] = X::mfma(rf[u][g][k], ho[k],
                                           k < NACC ? ((BIAS_C && k == 0) ? biasc[u][g] : f32x4{0.f, 0.f, 0.f, 0.f}) : accp[k % NACC][u][g]);
        if (k % NACC == NACC - 1) __builtin_amdgcn_sched_barrier(0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (t > 0) {
      if (KW > 1) {
        bool fail;
        if constexpr (PAIRS) fail = ll_gather_pairs<T, NP>(rLL, (unsigned)((t - 1) & 1) * LLW * 8u, qpoll, t - 1, hbuf[cur], a.status, a.spin_limit, a.poll_delay, rot_w, OWN_FIRST ? LLW : 0);
        else fail = ll_gather<T, NP, M44>(llbase + (size_t)((t - 1) & 1) * LLW, qpoll, t - 1, hbuf[cur], a.status, a.spin_limit, a.poll_delay, rot_w, OWN_FIRST ? LLW : 0);
        if (barrier_or(fail, &dead_flag)) { dead = true; return; }
      } else {
        lds_barrier();
      }
    }
    FRNN_STAMP(c1);
    if constexpr (!WX_LATE) load_wx(wn, min(t + PD, Tn - 1));
    // resident decode kernel: the first probe for this token's Wx goes out here and comes back behind the MFMAs;
    // R h_(t-1) does not need it, so a token that arrives while the product runs costs its gate math only
    Dw<RI::DW> mrec[MB ? UTW : 1];
    const unsigned mslot = MB ? (unsigned)(t & (a.slots - 1)) : 0u;
    auto mb_probe = [&]() __attribute__((always_inline)) {
#pragma unroll
      for (int u = 0; u < (MB ? UTW : 0); ++u) mrec[u] = mb_load<RI::DW>(rIn, mi_v[u], mslot * (unsigned)a.in_slot);
    };
    if constexpr (MB) mb_probe();
    Dw<ND_> wcl[PW ? UTW : 1][PW ? GW : 1];  // this step's Wx from the producer wave's buffer
    if constexpr (PW) {
      // (the lane's E consecutive units of a gate: 2, 4 or 8 bytes)
      const T* const wb = wbuf + cur * WBUF;
#pragma unroll
      for (int u = 0; u < UTW; ++u)
#pragma unroll
        for (int g = 0; g < GW; ++g) {
          const T* const src = wb + (((w * UTW + u) * GW + g) * TR + brow) * 16 + esub;
          if constexpr (E == 1) wcl[u][g].v[0] = *reinterpret_cast<const unsigned short*>(src);
          else if constexpr (E == 2) wcl[u][g].v[0] = *reinterpret_cast<const unsigned*>(src);
          else { const uint2 v = *reinterpret_cast<const uint2*>(src); wcl[u][g].v[0] = v.x; wcl[u][g].v[1] = v.y; }
        }
    }

    // h fragments are read KC k-steps ahead of the MFMAs that use them, so LDS latency is paid once
    f32x4 acc[UTW][GR];
    float ry44[M44 ? UTW : 1][4];  // 4x4x1 form: the lane's element, gates 0..3
    if constexpr (M44) {
      const float* hf = reinterpret_cast<const float*>(hbuf[cur]) + lane + kh * DK * 4;  // (this wave's half of k)
      float ha[DK / 16];
#pragma unroll
      for (int v = 0; v < DK / 16; ++v) ha[v] = hf[64 * v];
      __builtin_amdgcn_sched_barrier(0);
      f32x4 ac[UTW][4];  // 4 independent accumulation chains per tile
#pragma unroll
      for (int v = 0; v < DK / 16; ++v) {
#pragma unroll
        for (int u = 0; u < UTW; ++u) mfma_4x4x1_bcast16(ha[v], &rb[u][16 * v], ac[u], v == 0);
      }
      f32x4 sum[UTW];
#pragma unroll
      for (int u = 0; u < UTW; ++u) {
        sum[u] = (ac[u][0] + ac[u][1]) + (ac[u][2] + ac[u][3]);
        if constexpr (KSP > 1) { if (kh != 0) psum[((wt * UTW + u) * (KSP - 1) + kh - 1) * 64 + lane] = sum[u]; }
      }
      // (the buffer is free again before the second wave's next write: the barrier of the next step's exchange wait,
      // which every pair-split tiling has, lies in between)
      if constexpr (KSP > 1) lds_barrier();
#pragma unroll
      for (int u = 0; u < UTW; ++u) {
        if constexpr (KSP > 1) {
          if (kh == 0) {
#pragma unroll
            for (int i = 0; i < KSP - 1; ++i) sum[u] += psum[((wt * UTW + u) * (KSP - 1) + i) * 64 + lane];
          }
        }
        // lane 4*blk + j holds (gate j, unit blk) of batch rows 0..3; after the transpose lane 4*blk + b holds
        // gates 0..3 of (batch row b, unit blk): the element that Own<4> gives this lane
        ry44[u][0] = sum[u][0]; ry44[u][1] = sum[u][1]; ry44[u][2] = sum[u][2]; ry44[u][3] = sum[u][3];
        quad_transpose(ry44[u], lane);
      }
    }
    if constexpr (!M44) {
    // (the own k-steps are done; wave pairs that split k: this wave's half of h)
    const Frag* hf = reinterpret_cast<const Frag*>(hbuf[cur]) + lane + KSO * 64 + (KS16 ? kh * KSW * 64 : 0);
    constexpr int KS = KSW;  // (k-steps of this wave, in this block)
    constexpr int KC = chunk_of(KS - KSO);
    static_assert((KS - KSO) % KC == 0, "k-steps must split into whole chunks");
    Frag hq[2][KC];
#pragma unroll
    for (int k = 0; k < KC; ++k) hq[0][k] = hf[k * 64];
    Frag la_next[UTW][GR];
    if constexpr (RLK > 0 && KSR == 0) {
#pragma unroll
      for (int u = 0; u < UTW; ++u)
#pragma unroll
        for (int g = 0; g < GR; ++g) la_next[u][g] = rl[(u * GR + g) * 64];
    }
    // keep the reads up here: issued just in time they would expose the LDS latency once per chunk
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int kc = 0; kc < (KS - KSO) / KC; ++kc) {
      if (kc + 1 < (KS - KSO) / KC) {
#pragma unroll
        for (int k = 0; k < KC; ++k) hq[(kc + 1) & 1][k] = hf[((kc + 1) * KC + k) * 64];
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int k = 0; k < KC; ++k) {
        const int ks = KSO + kc * KC + k, j = ks % NACC;
        // fragments kept in LDS: those of the next k-step are requested before this one's MFMAs
        Frag la[UTW][GR];
        if constexpr (RLK > 0) {
          if (ks >= KSR) {
#pragma unroll
            for (int u = 0; u < UTW; ++u)
#pragma unroll
              for (int g = 0; g < GR; ++g) la[u][g] = la_next[u][g];
          }
          if (ks + 1 >= KSR && ks + 1 < KS) {
#pragma unroll
            for (int u = 0; u < UTW; ++u)
#pragma unroll
              for (int g = 0; g < GR; ++g) la_next[u][g] = rl[(((ks + 1 - KSR) * UTW + u) * GR + g) * 64];
            __builtin_amdgcn_sched_barrier(0);
          }
        }
#pragma unroll
        for (int u = 0; u < UTW; ++u)
#pragma unroll
          for (int g = 0; g < GR; ++g)
            accp[j][u][g] = X::mfma(ks < KSR ? rf[u][g][ks < KSR ? ks : 0] : la[u][g], hq[kc & 1][k],
                                    ks < NACC ? ((BIAS_C && ks == 0) ? biasc[u][g] : f32x4{0.f, 0.f, 0.f, 0.f}) : accp[j][u][g]);
        // group by group: consecutive MFMAs then never depend on each other
        if (j == NACC - 1) __builtin_amdgcn_sched_barrier(0);
      }
    }
#pragma unroll
    for (int u = 0; u < UTW; ++u)
#pragma unroll
      for (int g = 0; g < GR; ++g) {
        acc[u][g] = accp[0][u][g];
#pragma unroll
        for (int j = 1; j < NACC; ++j) acc[u][g] += accp[j][u][g];
      }
    if constexpr (KS16) {
      // the second wave of a pair hands its accumulators over (the buffer is free again before its next write: the
      // barrier of the next step's exchange wait lies in between)
#pragma unroll
      for (int u = 0; u < UTW; ++u)
#pragma unroll
        for (int g = 0; g < GR; ++g) { if (kh != 0) psum[((wt * UTW + u) * GR + g) * 64 + lane] = acc[u][g]; }
      lds_barrier();
#pragma unroll
      for (int u = 0; u < UTW; ++u)
#pragma unroll
        for (int g = 0; g < GR; ++g) { if (kh == 0) acc[u][g] += psum[((wt * UTW + u) * GR + g) * 64 + lane]; }
    }
    }  // !M44

    if constexpr (WX_LATE) {
      load_wx(wn, min(t + PD, Tn - 1));
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (MB) {
      // wait for the token: every record of this wave's valid lanes carries the tags of token t.  Bounded: after
      // idle_limit probes, or when the stop word is set, the workgroup leaves the loop (all waves together, behind
      // one barrier) and the kernel ends normally
      int give_up = a.spin_limit < -1 ? MB_END_IDLE : MB_END_NONE;  // (host-side test hook: give up at once)
      for (int spins = 0; give_up == MB_END_NONE; ++spins) {
        bool ok = true;
#pragma unroll
        for (int u = 0; u < UTW; ++u) ok = ok & (!bvalid | mb_ok<T, GW>(mrec[u], t));
        if (__all(ok)) break;
        if (spins > a.idle_limit) { give_up = MB_END_IDLE; break; }
        if ((spins & 15) == 15 && __any(__hip_atomic_load(mb_ctrl + MB_STOP, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)) {
          give_up = MB_END_STOP; break;
        }
        mb_probe();
      }
      if (give_up != MB_END_NONE && lane == 0) stop_reason = give_up;
      if (barrier_or(give_up != MB_END_NONE, &stop_flag)) { stopped = true; return; }
    }
#ifdef FRNN_TRACE
    { float sink = 0.f;
#pragma unroll
      for (int u = 0; u < UTW; ++u)
#pragma unroll
        for (int g = 0; g < GR; ++g) sink += M44 ? ry44[u][g] : acc[u][g][0];
      asm volatile("" ::"v"(sink)); }
#endif
    FRNN_STAMP(c2);
    if (KSP == 1 || kh == 0) {  // (wave-uniform: the second wave of a pair has handed its sums over)
#pragma unroll
    for (int u = 0; u < UTW; ++u) {
      float ryv[GR][E], wxv[GW][E];
#pragma unroll
      for (int g = 0; g < GR; ++g) {
        if constexpr (M44) ryv[g][0] = ry44[u][g];
        else own_elems<TR>(acc[u][g], ryv[g]);
        if constexpr (!BIAS_C) {
#pragma unroll
          for (int e = 0; e < E; ++e) ryv[g][e] += bown[u][g][e];
        }
      }
#pragma unroll
      for (int g = 0; g < GW; ++g) {
        if constexpr (MB) wxv[g][0] = mb_value<T, GW>(mrec[u], g);
        else unpack<E>(PW ? wcl[PW ? u : 0][PW ? g : 0] : wc[u][g], wxv[g], (T*)0);
      }
      float cv[NCA][E];
      float so[S][E];
#pragma unroll
      for (int e = 0; e < E; ++e) {
        float ry[GR], wx[GW], cc[NCA];
#pragma unroll
        for (int g = 0; g < GR; ++g) ry[g] = ryv[g][e];
#pragma unroll
        for (int g = 0; g < GW; ++g) wx[g] = wxv[g][e];
        if constexpr (CXS >= 0) cc[NC] = s[u][e][CXS];  // (before the step overwrites it)
        CM::fwd(ry, wx, bx[u][e], s[u][e], cc);
        s[u][e][0] = clamp_if(s[u][e][0], a.h_clip);
#pragma unroll
        for (int c = 0; c < NCX; ++c) cv[c][e] = cc[c];
#pragma unroll
        for (int k = 0; k < S; ++k) so[k][e] = s[u][e][k];
      }
      // the new h first: it is what the next step (of every workgroup of the head) waits for
      // (the own slice goes straight to the LDS buffer of the next step: the workgroup does not poll it)
      if (KW > 1) ll_write<E>((T*)0, llbase, (unsigned)(bvalid ? (t & 1) : 2) * (unsigned)(LLW * 8), brow, ub[u] + esub, so[0], t, near_m);
      if constexpr (M44) reinterpret_cast<float*>(hbuf[cur ^ 1])[lds_index4(brow, ub[u] + esub)] = so[0][0];
      else lds_write<E>(hbuf[cur ^ 1], brow, ub[u] - rot_u + esub, so[0]);
      if constexpr (MB) {  // the new states of the element as one tagged record of the outbox
        unsigned sbits[S];
#pragma unroll
        for (int k = 0; k < S; ++k) sbits[k] = mb_bits<T>(so[k][0]);
        mb_store<RO::DW>(mb_pack<T, S>(sbits, t), rOut, mo_v[u], mslot * (unsigned)a.out_slot);
      } else if constexpr (PST) {  // outputs to LDS as they lie in memory; the producer wave stores them one step later
        static_assert(!PST || E == 1, "producer-wave stores: 4-row tiles");
        T* const ob = obuf + cur * OB;
#pragma unroll
        for (int k = 0; k < S; ++k)
          *reinterpret_cast<unsigned short*>(ob + (k * TR + brow) * OBR + ub[u] + esub) = (unsigned short)pack<E>(so[k], (T*)0).v[0];
        if constexpr (NC > 0) {
          const Dw<NWC> cw = cache_pack<T, NCA, E>(cv);
          unsigned* const dst = reinterpret_cast<unsigned*>(ob + OB_ST + (((w * UTW + u) * TR + brow) * 16 + (esub & 15)) * NCP);
          if constexpr (NWC == 2) *reinterpret_cast<uint2*>(dst) = make_uint2(cw.v[0], cw.v[1]);
          else {
#pragma unroll
            for (int i = 0; i < NWC; ++i) dst[i] = cw.v[i];
          }
        }
      } else {
#pragma unroll
      for (int k = 0; k < S; ++k)
        buf_store<ND_, SB>(pack<E>(so[k], (T*)0), rSt, st_v[u], ((unsigned)k * BS * Tn + t) * ND * ES);
      // private cache layout [t][head][unit tile][batch row][16 units][value]: one store per tile
      if constexpr (NC > 0)
        buf_store_wide<NWC>(cache_pack<T, NCA, E>(cv), rCa, ca_v[u], (((unsigned)t * N + n) * (D / 16)) * Bpad * 16 * NCP * ES);
      }
    }
    }
#ifdef FRNN_TRACE
    FRNN_STAMP(c3);
    tr[0] += c1 - c0; tr[1] += c2 - c1; tr[2] += c3 - c2;
#endif
  };

  // the time loop, unrolled over the ring: step t + j consumes set j and refills the set that the
  // step before it consumed
  int t = 0;
  int served = 0;  // resident decode kernel: tokens whose states were posted
  if constexpr (MB) {
    for (; t < Tn && !dead; ++t) {
      step(t, wx[0], wx[0]);
      if (dead || stopped) break;
      served = t + 1;
    }
    t = Tn;
  }
  if constexpr (!MB && PD == 1) {
    // (written out: the general form below changes the register allocation of kernels that sit
    // at the register limit)
    for (; t + 1 < Tn && !dead; t += 2) {
      step(t, wx[0], wx[1]);
      if (dead) break;
      step(t + 1, wx[1], wx[0]);
    }
    if (!dead && t < Tn) step(t, wx[0], wx[1]);
    t = Tn;
  }
  for (; !MB && t + PD < Tn && !dead; t += PD + 1) {
#pragma unroll
    for (int j = 0; j <= PD; ++j) {
      step(t + j, wx[j], wx[(j + PD) % (PD + 1)]);
      if (dead) break;
    }
  }
#pragma unroll
  for (int j = 0; j < PD; ++j)
    if (!MB && !dead && t + j < Tn) step(t + j, wx[j], wx[(j + PD) % (PD + 1)]);

  if constexpr (PST) lds_barrier();  // (the last step's outputs are in LDS: the producer wave stores them behind this barrier)
#ifdef FRNN_TRACE
  if (lane == 0 && a.trace) {
    long long* o = a.trace + ((size_t)blockIdx.x * WAVES + w) * 4;
    o[0] = tr[0]; o[1] = tr[1]; o[2] = tr[2]; o[3] = clock64() - tr_begin;
  }
#endif
  if (a.carry && bvalid) {
#pragma unroll
    for (int u = 0; u < UTW; ++u)
#pragma unroll
      for (int e = 0; e < E; ++e)
#pragma unroll
        for (int k = 0; k < S; ++k) a.carry[((size_t)k * B + bg) * ND + (size_t)n * D + ub[u] + esub + e] = s[u][e][k];
  }
  if constexpr (MB) {
    // (a resident kernel reports through the control block of its mailbox; the caller's collecting kernel marks what it
    // did not get)
    if (tid == 0 && dead) __hip_atomic_store(a.status, (int)STATUS_WAIT_EXPIRED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (tid == 0 && grp == 0 && slice == 0) {
      __hip_atomic_store(mb_ctrl + MB_DONE, served, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(mb_ctrl + MB_REASON, dead ? (int)MB_END_WAIT : stopped ? stop_reason : (int)MB_END_TOKENS,
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return;
  }
  if (dead) {
    // bounded wait ran out: report, and make the damage visible (NaN in every h of this
    // workgroup's units; the step that failed is not known exactly, so all steps are marked)
    if (tid == 0) __hip_atomic_store(a.status, (int)STATUS_WAIT_EXPIRED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    float nanv[E];
#pragma unroll
    for (int e = 0; e < E; ++e) nanv[e] = __uint_as_float(0x7fc00000u);
    for (int tt = 0; tt < Tn; ++tt)
#pragma unroll
      for (int u = 0; u < UTW; ++u) buf_store<ND_, SB>(pack<E>(nanv, (T*)0), rSt, st_v[u], (unsigned)tt * ND * ES);
  }
}

}  // namespace frnn
