// Fused backward: one persistent kernel runs the reverse scan over all T steps.
//
// Replaces FLASHRNNCellFusedBackward, flashrnn/flashrnn/fused/flashrnn_fused_backward.cu:129-624
// and gradientBiasAggregationKernel (:626-665; the bias sums are kept in registers across T here).
//
// Same ownership as the forward kernel: a lane owns 4 units x 1 batch row of UTW unit tiles, and
// the KW workgroups of a (head, batch tile) group own D/KW units each.
// One reverse step t:
//   gate cache, s_{t-1}, s_t and the upstream cotangent of s_t (prefetched one step ahead)
//   -> per-element adjoint -> dg_t of the OWN units; dWx_t stored in the public layout; db summed
//      in registers
//   -> own dg_t (16 x G_r*D/KW, storage type) to LDS in fragment order, one workgroup barrier
//   -> MFMA over the own gate rows only (the contraction is split between the workgroups, the
//      reference's optional d_state_buffer scheme, flashrnn_fused_backward.cu:510-553):
//        part[p] = sum_{k own} Rt[p][k] dg_t[k]   for ALL previous units p of the head,
//      A = rows p of the transposed R, resident in registers
//   -> wave w keeps the partial sums of the tiles it owns itself and sends the others, as tagged
//      fp32 words, to wave w of the owning workgroup; it then polls its own inbox for the KW-1
//      partial sums of its tiles and adds everything to the running cotangent dh_{t-1}.
// Exchanging partial dh (D values per row) instead of dg (G_r*D values per row) moves 2-4x
// fewer bytes through L2 per step.
#pragma once
#include <type_traits>
#include "frnn_exchange.h"
#include "frnn_fused_fwd.h"
#include "frnn_pointwise.h"


namespace frnn {

#ifndef FRNN_STAMP
#ifdef FRNN_TRACE
#define FRNN_STAMP(var) __builtin_amdgcn_sched_barrier(0); const long long var = clock64(); __builtin_amdgcn_sched_barrier(0)
#else
#define FRNN_STAMP(var)
#endif
#endif

struct BwdArgs {
  const void* Rt;  // [N][D (previous unit p)][G_r*D (k = g*D + d)]
  const void* s0; const void* states; const void* cache; const void* dstates;
  void* dWx;       // [B,T,G_w,N,D]
  void* dgx;       // [B,T,N,D]: cotangent of R-side gates that have no Wx slot (gru: g); else null
  void* ds0;       // [S,B,N,D]
  float* dbp;      // [batch tiles][G_t][N][D] partial bias sums
  u64* ll; int* status;
  int* xcd;        // 32 words per group for xcd_handshake (zero at launch), or null: exchange stores stay agent scope
  int B, T, N;
  int BS;  // rows between the state planes of s0, states, dstates and ds0 ([S, BS, ...]); B unless the call covers a range of a larger batch
  int grp0, groups, groups_total, tile_rows;
  int spin_limit, poll_delay;
  float g_clip;  // > 0: cotangent carried into h_t clamped to [-g_clip, g_clip] (gradient_recurrent_clipval)
  int cut;       // != 0: no gradient through R h (gradient_recurrent_cut)
  long long* trace;  // phase cycle sums per wave; only written by -DFRNN_TRACE builds
  // recompute mode (kernels instantiated with RC = true): no gate cache; the gates of step t are rebuilt from
  // Wx_t, b and R h_(t-1), with h_(t-1) read back from the stored states
  const void* Wx; const void* R; const void* b;
  int pst;  // host side only: launch the instantiation whose producer wave stores dWx (bwd_producer_stores)
};

// words (64-bit for fp32 storage, 32-bit otherwise) of one inbox area of one group:
// [dst wg][wave][tile][src wg][element 4][lane 64]
constexpr size_t bwd_inbox_words(int D, int KW) { return (size_t)KW * (D / 16) * 256; }

// Resident operand of the reverse product: a wave holds KW*UTW*KS fragments of the transposed R (all
// destination tiles at its position, its workgroup's gate rows).  At 4 waves per workgroup a wave has
// 512 registers; when the fragments alone would take more than 288 of them (LSTM D = 768: 384), those
// of the last RLD destination tiles (as many as bring the rest down to 256) live in LDS instead (the reverse kernel needs little LDS otherwise)
// and are read back, one k-step ahead, as the A operand of their MFMAs.
constexpr int bwd_lds_tiles(int GR, int D, int WAVES, int UTW, int KW, int esize) {
  const int KM = esize == 4 ? 4 : 32, FR = esize == 4 ? 1 : 4;
  const int KS = GR * (D / KW) / KM, regs = KW * UTW * KS * FR, per = UTW * KS * FR;
  if (!(WAVES <= 4 && regs > 288)) return 0;
  const int want = (regs - 256 + per - 1) / per;
  // what fits: 160 KB of LDS minus the two dg buffers and some slack
  const int FRB = esize == 4 ? 4 : 16;
  const int room = (160 * 1024 - 2 * 16 * GR * (D / KW) * esize - 2048) / (WAVES * UTW * KS * 64 * FRB);
  // more than 8 remote destinations are processed in groups of 4 (see the kernel): whole groups in LDS
  if (KW - 1 > 8) return (want + 3) / 4 * 4 < room / 4 * 4 ? (want + 3) / 4 * 4 : room / 4 * 4;
  return want < room ? want : room;
}
constexpr size_t bwd_lds_bytes(int GR, int D, int WAVES, int UTW, int KW, int esize, bool rc = false) {
  const int KM = esize == 4 ? 4 : 32, FRB = esize == 4 ? 4 : 16;
  const int KS = GR * (D / KW) / KM;
  return (size_t)2 * 16 * GR * (D / KW) * esize + (size_t)WAVES * bwd_lds_tiles(GR, D, WAVES, UTW, KW, esize) * UTW * KS * 64 * FRB +
         (rc ? (size_t)2 * 16 * D * esize : 0);  // recompute mode: two buffers for h_(t-1) of the whole head
}

template <typename T> __device__ __forceinline__ typename ST<T>::Frag load_frag_at(const T* p);
template <> __device__ __forceinline__ bf16x8 load_frag_at<bf16_t>(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }
template <> __device__ __forceinline__ f16x8 load_frag_at<half_t>(const half_t* p) { return *reinterpret_cast<const f16x8*>(p); }
template <> __device__ __forceinline__ float load_frag_at<float>(const float* p) { return *p; }

// RC = true: recompute mode.  Nothing is cached by the forward pass; the reverse scan rebuilds the gates of
// step t-1 while the partial sums of step t travel between the workgroups (the rebuild does not depend on
// the running cotangent, so it is off the chain of dependent steps): h_(t-2) of the whole head comes back
// from the stored states (a few bytes per thread, fetched two steps ahead) into LDS, the forward product
// R h_(t-2) of the own units runs on MFMA with R resident beside R^T, and the forward gate math yields what
// the cache would have held.  For the sLSTM the stabilised gates exp(i - m') and exp(logsig(f) + m - m')
// are rebuilt from the stored (rounded) m_(t-2); the larger of the two is still exactly 1, the other carries
// the rounding error of m_(t-2) as a relative error (2^-9 |m| for bf16).
template <int F, typename T, int D, int WAVES, int UTW, int KW, int TR, bool RC = false, bool PSTV = false>
__global__ void __launch_bounds__((WAVES + (bwd_producer_wave(Cell<F>::GR, Cell<F>::NC, D, WAVES, UTW, KW, TR, (int)sizeof(T), RC) ? 1 : 0)) * 64)
fused_bwd_kernel(const BwdArgs a) {
  typedef Cell<F> C;
  typedef ST<T> X;
  typedef CellMath<F, X::FAST> CM;
  typedef typename X::Frag Frag;
  typedef Own<TR> O;
  constexpr int GR = C::GR, GW = C::GW, GT = C::GT, S = C::S, NC = C::NC;
  // (DSP = 2: pairs of waves share a tile position and split the destinations between them, see bwd_dest_split)
  constexpr int DSP = bwd_dest_split(GR, D, WAVES, UTW, KW, TR, (int)sizeof(T), RC), NPOS = WAVES / DSP;
  constexpr int NT = WAVES * 64, UT_WG = NPOS * UTW;
  static_assert(UT_WG * KW * 16 == D, "tiling must cover the head");
  constexpr int DL = D / KW;            // units owned by this workgroup
  constexpr int KDL = GR * DL;          // contraction length handled by this workgroup
  constexpr int KS = KDL / X::KM;
  static_assert(KDL % X::KM == 0 && DL % 8 == 0, "own gate rows must fill whole k-steps");
  constexpr int KE = X::KM / 4;         // consecutive k held by one lane of a fragment
  // (values per element of a cache line: the cell's NC and, where cache_carried_state says so, one state of step t-1)
  constexpr int CXS = RC ? -1 : cache_carried_state(F, (int)sizeof(T), D), NCX = NC + (CXS >= 0 ? 1 : 0);
  constexpr int NCA = NCX > 0 ? NCX : 1;
  // remote sources polled together: every round of polling costs at least one trip to L2 and back,
  // so as few rounds as 16 words per lane and probe allow, of equal size (no dummy loads)
  // (16 words per lane and probe; 32 for the 16-bit kernels at 8- and 16-row tiles, 2 and 4 words per source, where the
  // rounds halve: reverse kernel, B256 T512, GRU D = 1024 3.44 -> 3.18 ms, sLSTM D = 768 1.43 -> 1.37, LSTM D = 640 1.85 -> 1.83,
  // D = 512 1.04 -> 1.03, D = 768 no change; not the kernels whose wave pairs share the receive: LSTM D = 1024 1.54 -> 1.62)
  constexpr int RCW = sizeof(T) == 2 && TR >= 8 && DSP == 1 ? 32 : 16;
  constexpr int RC_MAX = RCW / (UTW * (TR / 4)) > 0 ? RCW / (UTW * (TR / 4)) : 1;
  constexpr int ROUNDS = KW == 1 ? 1 : (KW - 1 + RC_MAX - 1) / RC_MAX;
  constexpr int PSRC = KW == 1 ? 1 : (KW - 1 + ROUNDS - 1) / ROUNDS;  // sources polled per round
  constexpr size_t INW = bwd_inbox_words(D, KW);
  // Waves that split the destinations of a tile position (DSP > 1) also split its sources where one wave would poll them
  // in several rounds, each a trip to memory and back: wave hf polls sources 1 + hf * SRC_W .. and hands its sum to the
  // first wave through LDS.  Measured, reverse kernel, 1024 steps: LSTM fp32 D = 1024 (63 sources at agent scope, 4 rounds of
  // 16 become one per wave) 8.68 -> 6.30 ms, bf16 D = 1024 B16 2.67 -> 2.39; also from 13 sources on, where one round
  // shrinks to half the words: fp32 D = 512 2.62 -> 2.52, D = 448 2.61 -> 2.55 (D = 384, 11 sources: 2.49 -> 2.54, left alone).
  constexpr bool RSP = DSP > 1 && (ROUNDS > 1 || KW >= 14);
  constexpr int SRC_W = RSP ? (KW - 1 + DSP - 1) / DSP : 1;                    // sources per wave
  constexpr int ROUNDS_W = (SRC_W + RC_MAX - 1) / RC_MAX, PSRC_W = (SRC_W + ROUNDS_W - 1) / ROUNDS_W;
  constexpr int E = O::E, ND_ = NDW<T, E>::value;
  constexpr bool SB = NDW<T, E>::SUB;  // single bf16 elements: 16-bit memory operations
  constexpr unsigned ES = sizeof(T);
  // fp32, 4-row batch tiles, several workgroups per head: the product runs on v_mfma_f32_4x4x1_16B_f32 with the 4
  // batch rows on the 4-wide side (see the forward kernel).  Block = previous unit p of a destination tile, the 4
  // columns of a block = 4 destination workgroups (the wave's tile position in each), A = dg of the own gate rows
  // (the values of one block broadcast to all 16), one instruction per k: KDL instructions of 8 cycles per 4
  // destinations instead of KDL / 4 of 32 per destination.
  constexpr int NG4 = (KW + 3) / 4;  // groups of 4 destinations
  constexpr int NGH = (NG4 + DSP - 1) / DSP;  // of them per wave: group qq of wave half hf is group qq * DSP + hf
  // (the whole operand, a register per destination group and own gate row, in the registers of a wave: wherever the
  // 16x16x4 form keeps it there too, and up to 320 registers at one wave per SIMD)
  constexpr bool M44 = sizeof(T) == 4 && TR == 4 && KW >= 2 && !RC &&
                       (bwd_lds_tiles(GR, D, WAVES, UTW, KW, (int)sizeof(T)) == 0 || (WAVES <= 4 && NGH * UTW * KDL <= 320));
  constexpr bool DS16 = DSP > 1 && sizeof(T) == 2;  // 16-bit kernels whose wave pairs split the destinations
  constexpr int NL = DS16 ? KW / DSP : KW;          // destinations whose fragments a wave keeps: hf * NL .. hf * NL + NL - 1
  static_assert(DSP == 1 || M44 || DS16, "destinations are split between wave pairs in these two forms only");

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* const gbuf0 = reinterpret_cast<T*>(smem_raw);
  T* const gbuf1 = gbuf0 + 16 * KDL;
  constexpr int RLD = DS16 ? 0 : bwd_lds_tiles(GR, D, WAVES, UTW, KW, (int)sizeof(T)), KWR = NL - RLD;
  // this lane's fragments of the last RLD destination tiles: [wave][tile][u][ks][lane]
  Frag* const rl = reinterpret_cast<Frag*>(smem_raw + (size_t)2 * 16 * KDL * sizeof(T)) +
                   (size_t)(threadIdx.x >> 6) * RLD * UTW * KS * 64 + (threadIdx.x & 63);
  // recompute mode: h_(t-1) of the whole head, 16 x D in fragment order, two buffers (behind the R^T tiles)
  constexpr int KSF = D / X::KM;   // k-steps of the forward product
  T* const hb0 = reinterpret_cast<T*>(smem_raw + bwd_lds_bytes(GR, D, WAVES, UTW, KW, (int)sizeof(T)));
  T* const hb1 = hb0 + 16 * D;
  // a static LDS word, not a slice of the dynamic array: through a pointer computed from the
  // dynamic array the compiler reads the flag with a flat load, which has to wait for every global
  // load in flight (measured: the operand prefetch's full HBM latency, once per step)
  __shared__ int dead_flag_word, near_word;
  int* const dead_flag = &dead_flag_word;
  __shared__ float rsum[RSP ? NPOS * (DSP - 1) * UTW * O::E * 64 : 1];  // sums of the sources polled by the other waves: [position][wave - 1][tile][element][lane]

  int grp_l, slice;
  if (!decode_block(a.groups, KW, grp_l, slice)) return;
  const int grp = a.grp0 + grp_l;
  const int N = a.N, Tn = a.T, B = a.B, BS = a.BS;
  const int n = grp % N, bt = grp / N;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int r16 = lane & 15, q4 = lane >> 4;
  const int brow = O::row(r16), esub = O::sub(r16, q4);
  const int bg = bt * TR + brow;
  const unsigned Bpad = (unsigned)a.B;  // rows of the gate cache: padded rows are never read or written
  // wave w of a pair-split workgroup: tile position w / 2, destination groups of parity w % 2; the lanes of a second
  // wave own no element (every load of theirs returns zero, every store is dropped)
  const int w_u = __builtin_amdgcn_readfirstlane(w);
  const int hf = DSP > 1 ? w_u % DSP : 0, wp = DSP > 1 ? w_u / DSP : w, wp_u = DSP > 1 ? w_u / DSP : w_u;
  const bool rvalid = bg < B, bvalid = rvalid && hf == 0;
  const T* __restrict__ Rt = static_cast<const T*>(a.Rt);
  const unsigned ND = (unsigned)N * D;

  const rsrc_t rSt = make_rsrc(a.states, ((size_t)(S - 1) * BS + B) * Tn * ND * ES);
  const rsrc_t rS0 = make_rsrc(a.s0, ((size_t)(S - 1) * BS + B) * ND * ES);
  const rsrc_t rDs = make_rsrc(a.dstates, ((size_t)(S - 1) * BS + B) * Tn * ND * ES);
  constexpr int NCP = CacheBlk<T, NCA>::NCP, NWC = CacheBlk<T, NCA>::template Words<E>::value;
  const rsrc_t rCa = make_rsrc(a.cache, (size_t)Tn * N * Bpad * D * (NC ? NCP : 0) * ES);
  const rsrc_t rDw = make_rsrc(a.dWx, (size_t)B * Tn * GW * ND * ES);
  const rsrc_t rDx = make_rsrc(a.dgx, (size_t)B * Tn * ND * ES);
  const rsrc_t rWx = make_rsrc(a.Wx, RC ? (size_t)B * Tn * GW * ND * ES : 0);

  // ---- the producer wave (see bwd_producer_wave): the workgroup's last wave.  It takes part in every barrier of the
  //      compute waves, in the same order and under the same conditions (wave-uniform values that every wave reads from
  //      LDS behind a barrier, and kernel arguments).  Iterations count the reverse steps: iteration i is step
  //      T-1-i.  The operands of iteration j travel in register set j % 3; during iteration i the compute waves read
  //      those of iteration i+1 from buffer (i+1) & 1 (behind the barrier of the step) and this wave writes those of
  //      iteration i+2 into the other buffer and sends for those of iteration i+4 --------------------------------------
  constexpr bool PW = bwd_producer_wave(GR, NC, D, WAVES, UTW, KW, TR, (int)sizeof(T), RC);
  // one buffer: [cache: tile][row][16 units][NCP values] [s_(t-1): state][tile][row][16 units] [cotangent: the same]
  constexpr int PB_CA = NC > 0 ? UT_WG * TR * 16 * NCP : 0, PB_ST = S * UT_WG * TR * 16, PB = PB_CA + 2 * PB_ST;
  static_assert(!PW || 2 * PB * (int)sizeof(T) + 16 == bwd_producer_bytes(NCX, S, UT_WG, TR, (int)sizeof(T)), "hand-over buffer size");
  // the carried state comes out of the cache line instead of a load of its own (the kernels with a producer wave keep the
  // load: it is the producer's, off the compute waves' chain)
  constexpr bool CXU = CXS >= 0 && !PW;
  T* const pbuf = reinterpret_cast<T*>(smem_raw + bwd_lds_bytes(GR, D, WAVES, UTW, KW, (int)sizeof(T)));
  // Producer-wave stores (PSTV instantiations, chosen on the host for launches that fill the device; see the forward
  // kernel): the compute waves leave dWx_t (and the GRU's g-gate cotangent) in LDS as they lie in memory, two buffers by
  // iteration parity behind the hand-over buffers, and the producer wave stores them in 16-byte pieces behind the
  // barrier of the step.
  constexpr bool PST = PSTV && bwd_producer_stores(GR, NC, D, WAVES, UTW, KW, TR, (int)sizeof(T), RC);
  constexpr int DBR = D + 8;  // (row stride: see the forward kernel)
  constexpr int DB_W = GW * TR * DBR, DB_X = F == FRNN_GRU ? TR * DBR : 0, DB = DB_W + DB_X;  // [gate][row][unit] [row][unit]
  static_assert(!PST || DB * 2 * (int)sizeof(T) == bwd_producer_store_bytes(GW, F == FRNN_GRU, D, TR, (int)sizeof(T)), "dWx hand-over size");
  T* const dbuf = pbuf + 2 * PB + 8;
  if constexpr (PW) {
    if (w == WAVES) {
      constexpr int CPR = NCP * 2;  // 16-byte pieces per (tile, batch row) of the cache
      constexpr int CP_TOT = NC > 0 ? UT_WG * TR * CPR : 0, NPC = (CP_TOT + 63) / 64;
      constexpr int SP_TOT = S * UT_WG * TR * 2, NPS = (SP_TOT + 63) / 64;  // pieces of 8 units of one state, tile and row
      unsigned cvo[NPC > 0 ? NPC : 1], svo[NPS], spo[NPS], s0o[NPS]; int cl[NPC > 0 ? NPC : 1], sl[NPS];
#pragma unroll
      for (int i = 0; i < NPC; ++i) {
        const int c = lane + 64 * i, q = c % CPR, pr = (c / CPR) % TR, ptile = c / (CPR * TR);
        const bool ok = c < CP_TOT && bt * TR + pr < B;
        cvo[i] = ok ? ((((unsigned)(slice * UT_WG + ptile) * Bpad + bt * TR + pr) * 16) * NCP * ES + q * 16) : kInvalidOff;
        cl[i] = c < CP_TOT ? ((ptile * TR + pr) * 16) * NCP + q * 8 : -1;
      }
#pragma unroll
      for (int i = 0; i < NPS; ++i) {
        const int c = lane + 64 * i, half = c & 1, pr = (c >> 1) % TR, ptile = ((c >> 1) / TR) % UT_WG, pk = (c >> 1) / (TR * UT_WG);
        const bool ok = c < SP_TOT && bt * TR + pr < B;
        const unsigned col = n * D + slice * DL + ptile * 16 + half * 8;
        // (planes that the cell's adjoint never reads: out of range, no memory traffic; their LDS slots hold zeros)
        const bool oks = ok && ((C::SPM >> pk) & 1), okd = ok && ((C::DSM >> pk) & 1);
        svo[i] = okd ? ((((unsigned)(pk * BS + bt * TR + pr) * Tn) * ND + col) * ES) : kInvalidOff;   // + t * ND * ES
        spo[i] = oks ? ((((unsigned)(pk * BS + bt * TR + pr) * Tn) * ND + col) * ES) : kInvalidOff;
        s0o[i] = oks ? (((unsigned)(pk * BS + bt * TR + pr) * ND + col) * ES) : kInvalidOff;
        sl[i] = c < SP_TOT ? ((pk * UT_WG + ptile) * TR + pr) * 16 + half * 8 : -1;
      }
      struct Ops { Dw<4> ca[NPC > 0 ? NPC : 1], sp[NPS], dso[NPS]; };
      Ops set[3];
      auto fetch = [&](Ops& o, int j) __attribute__((always_inline)) {
        const int t = Tn - 1 - j > 0 ? Tn - 1 - j : 0;  // (beyond the last step: the operands of step 0 again, unused)
        const bool first = t == 0;
        const rsrc_t rPrev = first ? rS0 : rSt;
#pragma unroll
        for (int i = 0; i < NPC; ++i) o.ca[i] = buf_load<4>(rCa, cvo[i], (((unsigned)t * N + n) * (D / 16)) * Bpad * 16 * NCP * ES);
#pragma unroll
        for (int i = 0; i < NPS; ++i) {
          o.dso[i] = buf_load<4>(rDs, svo[i], (unsigned)t * ND * ES);
          o.sp[i] = buf_load<4>(rPrev, first ? s0o[i] : spo[i], first ? 0u : (unsigned)(t - 1) * ND * ES);
        }
      };
      // (no branch on the lane: behind one the compiler waits for every load in flight, the latest ones included;
      // lanes without a piece write to the 16 spare bytes behind the buffers)
      auto put = [&](const Ops& o, int j) __attribute__((always_inline)) {
        T* const pb = pbuf + (j & 1) * PB;
        T* const spare = pbuf + 2 * PB;
#pragma unroll
        for (int i = 0; i < NPC; ++i)
          *reinterpret_cast<uint4*>(cl[i] >= 0 ? pb + cl[i] : spare) = make_uint4(o.ca[i].v[0], o.ca[i].v[1], o.ca[i].v[2], o.ca[i].v[3]);
#pragma unroll
        for (int i = 0; i < NPS; ++i) {
          *reinterpret_cast<uint4*>(sl[i] >= 0 ? pb + PB_CA + sl[i] : spare) = make_uint4(o.sp[i].v[0], o.sp[i].v[1], o.sp[i].v[2], o.sp[i].v[3]);
          *reinterpret_cast<uint4*>(sl[i] >= 0 ? pb + PB_CA + PB_ST + sl[i] : spare) = make_uint4(o.dso[i].v[0], o.dso[i].v[1], o.dso[i].v[2], o.dso[i].v[3]);
        }
      };
      // producer-wave stores: the 16-byte pieces of a step's dWx (and dgx) that this lane stores
      constexpr int WP_TOT = PST ? GW * TR * (D / 8) : 0, NWP = (WP_TOT + 63) / 64;
      constexpr int XP_TOT = PST && F == FRNN_GRU ? TR * (D / 8) : 0, NXP = (XP_TOT + 63) / 64;
      unsigned wvo[NWP > 0 ? NWP : 1], xvo[NXP > 0 ? NXP : 1]; int wl[NWP > 0 ? NWP : 1], xl[NXP > 0 ? NXP : 1];
#pragma unroll
      for (int i = 0; i < NWP; ++i) {
        const int c = lane + 64 * i, ch = c % (D / 8), pr = (c / (D / 8)) % TR, pg = c / ((D / 8) * TR);
        const bool ok = c < WP_TOT && bt * TR + pr < B;
        wvo[i] = ok ? ((((unsigned)(bt * TR + pr) * Tn * GW + pg) * ND + n * D + ch * 8) * ES) : kInvalidOff;  // + t * GW * ND * ES
        wl[i] = c < WP_TOT ? (pg * TR + pr) * DBR + ch * 8 : 0;
      }
#pragma unroll
      for (int i = 0; i < NXP; ++i) {
        const int c = lane + 64 * i, ch = c % (D / 8), pr = c / (D / 8);
        const bool ok = c < XP_TOT && bt * TR + pr < B;
        xvo[i] = ok ? (((unsigned)(bt * TR + pr) * Tn * ND + n * D + ch * 8) * ES) : kInvalidOff;  // + t * ND * ES
        xl[i] = c < XP_TOT ? DB_W + pr * DBR + ch * 8 : 0;
      }
      auto drain = [&](int i_) __attribute__((always_inline)) {  // dWx of iteration i_ (step T-1-i_), complete in dbuf[i_ & 1]
        const T* const db = dbuf + (i_ & 1) * DB;
        const unsigned t = (unsigned)(Tn - 1 - i_);
#pragma unroll
        for (int i = 0; i < NWP; ++i) {
          const uint4 v = *reinterpret_cast<const uint4*>(db + wl[i]);
          buf_store<4>(Dw<4>{{v.x, v.y, v.z, v.w}}, rDw, wvo[i], t * GW * ND * ES);
        }
#pragma unroll
        for (int i = 0; i < NXP; ++i) {
          const uint4 v = *reinterpret_cast<const uint4*>(db + xl[i]);
          buf_store<4>(Dw<4>{{v.x, v.y, v.z, v.w}}, rDx, xvo[i], t * ND * ES);
        }
      };
      fetch(set[1], 1); fetch(set[2], 2); fetch(set[0], 3);
      put(set[1], 1);
      __syncthreads();  // (the one of the prologue below)
      bool pdead = KW > 1 && __builtin_amdgcn_readfirstlane(near_word) < 0;
      if (!a.cut) {
        auto iter = [&](int i, const Ops& next, Ops& refill) __attribute__((always_inline)) {
          if (barrier_or(false, dead_flag)) { pdead = true; return; }
          put(next, i + 2);
#ifdef FRNN_PST_DRAIN_FIRST
          if constexpr (PST) drain(i);
          fetch(refill, i + 4);
#else
          fetch(refill, i + 4);  // (loads before stores: see the forward kernel)
          if constexpr (PST) drain(i);
#endif
        };
        int i = 0;
        for (; i + 2 < Tn && !pdead; i += 3) {
          iter(i, set[2], set[1]);
          if (pdead) break;
          iter(i + 1, set[0], set[2]);
          if (pdead) break;
          iter(i + 2, set[1], set[0]);
        }
        if (!pdead && i < Tn) {
          iter(i, set[2], set[1]);
          if (!pdead && i + 1 < Tn) iter(i + 1, set[0], set[2]);
        }
      }
      if (!pdead) barrier_or(false, dead_flag);  // (the one behind the time loop)
      return;
    }
  }

  int ub[UTW];
  unsigned wx_v[UTW], st_v[UTW], s0_v[UTW], ca_v[UTW];
#pragma unroll
  for (int u = 0; u < UTW; ++u) {
    ub[u] = (slice * UT_WG + wp * UTW + u) * 16;
    const unsigned d0 = n * D + ub[u] + esub;
    wx_v[u] = bvalid ? ((unsigned)bg * Tn * GW * ND + d0) * ES : kInvalidOff;
    st_v[u] = bvalid ? ((unsigned)bg * Tn * ND + d0) * ES : kInvalidOff;
    s0_v[u] = bvalid ? ((unsigned)bg * ND + d0) * ES : kInvalidOff;
    ca_v[u] = bvalid ? ((((unsigned)(ub[u] >> 4) * Bpad + bg) * 16 + (esub & 15)) * NCP) * ES : kInvalidOff;
  }

  // rtf[r][u][ks]: rows p of the tiles at this wave's position in workgroup (slice + r) % KW,
  // columns = the own gate rows, local index kk = g*DL + (d - slice*DL)
  constexpr int FRAG_REGS = (int)sizeof(Frag) / 4, RTF_REGS = KWR * UTW * KS * FRAG_REGS;
  constexpr int PIN_REGS = RC ? 0 : RTF_REGS > 160 ? (RTF_REGS < 232 ? RTF_REGS : 232) : 0;
  Frag rtf[KWR][UTW][KS];
  // 4x4x1 form: lane 4*blk + j holds row p = (tile of destination 4q + j, unit blk) of R^T, one register per own k
  float rtb[M44 ? NGH : 1][M44 ? UTW : 1][M44 ? KDL : 1];
  if constexpr (M44) {
    const int blk = lane >> 2, j = lane & 3;
#pragma unroll
    for (int q = 0; q < NGH; ++q) {
      const int r = 4 * (q * DSP + hf) + j;
      const int x = (slice + (r < KW ? r : 0)) % KW;
#pragma unroll
      for (int u = 0; u < UTW; ++u) {
        const float* row = reinterpret_cast<const float*>(Rt) + ((size_t)n * D + (x * UT_WG + wp * UTW + u) * 16 + blk) * (GR * D) + slice * DL;
#pragma unroll
        for (int kk = 0; kk < KDL; kk += 4) {
          const float4 v = *reinterpret_cast<const float4*>(row + (kk / DL) * D + (kk % DL));
          rtb[q][u][kk] = r < KW ? v.x : 0.f; rtb[q][u][kk + 1] = r < KW ? v.y : 0.f;
          rtb[q][u][kk + 2] = r < KW ? v.z : 0.f; rtb[q][u][kk + 3] = r < KW ? v.w : 0.f;
        }
      }
    }
#ifndef FRNN_NO_AGPR_PIN
    // what does not fit the architectural VGPRs beside the working set is pinned to accumulation registers, where the
    // MFMA reads it in place (left to the register allocator it is copied back before every use)
    // (384 registers: the 152 that would stay in VGPRs leave too little for the working set; left alone there)
    constexpr int ALL44 = NGH * UTW * KDL, PIN44 = ALL44 > 344 ? 0 : ALL44 - 112 > 232 ? 232 : ALL44 - 112;
#pragma unroll
    for (int q = 0; q < NGH; ++q)
#pragma unroll
      for (int u = 0; u < UTW; ++u)
#pragma unroll
        for (int kk = 0; kk < KDL; ++kk)
          if (ALL44 - 1 - ((q * UTW + u) * KDL + kk) < PIN44) asm volatile("" : "+a"(rtb[q][u][kk]));
#endif
  }
#pragma unroll
  for (int r = 0; r < (M44 ? 0 : NL); ++r) {
    const int x = (slice + hf * NL + r) % KW;  // (hf = 0 unless wave pairs split the destinations)
#pragma unroll
    for (int u = 0; u < UTW; ++u) {
      const T* row = Rt + ((size_t)n * D + (x * UT_WG + wp * UTW + u) * 16 + r16) * (GR * D) + slice * DL;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int kk0 = ks * X::KM + q4 * KE;
        const Frag f = load_frag_at<T>(row + (kk0 / DL) * D + (kk0 % DL));
        if (r < KWR) {
          rtf[r < KWR ? r : 0][u][ks] = f;
#ifndef FRNN_NO_AGPR_PIN
          // (see the forward kernel: resident fragments beyond what the architectural VGPRs hold are pinned to
          // the accumulation registers, where the MFMA reads them in place; in recompute mode the other operand
          // lives there instead)
          if constexpr (PIN_REGS > 0) {
            if (((r * UTW + u) * KS + (KS - 1 - ks)) * FRAG_REGS + FRAG_REGS <= PIN_REGS) asm volatile("" : "+a"(rtf[r][u][ks]));
          }
#endif
        }
        else rl[(((r - KWR) * UTW + u) * KS + ks) * 64] = f;
      }
    }
  }

  // recompute mode: rows of R of the own unit tiles (the forward kernel's resident operand) and the biases
  constexpr int GX = GT - GR > 0 ? GT - GR : 1;
  constexpr bool BIAS_C = O::E == 4;
  Frag rfw[RC ? UTW : 1][RC ? GR : 1][RC ? KSF : 1];
  f32x4 biasc[RC && BIAS_C ? UTW : 1][GR];
  float bown[RC ? UTW : 1][GR][BIAS_C ? 1 : O::E];
  float bxr[RC ? UTW : 1][O::E][GX];
  if constexpr (RC) {
    const T* __restrict__ Rm = static_cast<const T*>(a.R);
    const T* __restrict__ bias_g = static_cast<const T*>(a.b);
    typedef typename X::Vec4 Vec4;
#pragma unroll
    for (int u = 0; u < UTW; ++u) {
#pragma unroll
      for (int g = 0; g < GR; ++g) {
        const T* row = Rm + ((size_t)(g * N + n) * D + ub[u] + r16) * D;
#pragma unroll
        for (int ks = 0; ks < KSF; ++ks) {
          rfw[u][g][ks] = load_frag<T>(row, ks, q4);
#ifndef FRNN_NO_AGPR_PIN
          // R and R^T together exceed the 256 architectural VGPRs of a wave; this operand, which is used off
          // the chain of dependent steps, is the one to live in the accumulation registers, where the MFMA
          // reads it directly.  Left to the register allocator, fragments of both operands end up there as
          // spills, each copied back before its MFMA (measured: +400 cycles on the R^T product of a step)
          asm volatile("" : "+a"(rfw[u][g][ks]));
#endif
        }
        if constexpr (BIAS_C) {
          float v[4];
          unpack4<T>(*reinterpret_cast<const Vec4*>(bias_g + (size_t)(g * N + n) * D + ub[u] + q4 * 4), v);
          biasc[u][g] = f32x4{v[0], v[1], v[2], v[3]};
        } else {
#pragma unroll
          for (int e = 0; e < O::E; ++e) bown[u][g][e] = (float)bias_g[(size_t)(g * N + n) * D + ub[u] + esub + e];
        }
      }
#pragma unroll
      for (int e = 0; e < O::E; ++e)
#pragma unroll
        for (int g = GR; g < GT; ++g) bxr[u][e][g - GR] = (float)bias_g[(size_t)(g * N + n) * D + ub[u] + esub + e];
    }
  }

  // zero the LDS buffers once (rows beyond the tile are never written) and the flag
  for (int idx = tid; idx < (2 * 16 * KDL * (int)sizeof(T)) / 4; idx += NT) reinterpret_cast<unsigned*>(smem_raw)[idx] = 0u;
  if constexpr (RC) {
    for (int idx = tid; idx < (2 * 16 * D * (int)sizeof(T)) / 4; idx += NT) reinterpret_cast<unsigned*>(hb0)[idx] = 0u;
  }
  if (tid == 0) dead_flag_word = 0;
  // (as in the forward kernel: the status word of a call whose workgroups never wait is set here, not by a clearing kernel)
  if constexpr (KW == 1) { if (blockIdx.x == 0 && tid == 0) *a.status = 0; }

  float ds[UTW][E][S];
  float dbacc[UTW][E][GT];
#pragma unroll
  for (int u = 0; u < UTW; ++u)
#pragma unroll
    for (int e = 0; e < E; ++e) {
#pragma unroll
      for (int k = 0; k < S; ++k) ds[u][e][k] = 0.f;
#pragma unroll
      for (int g = 0; g < GT; ++g) dbacc[u][e][g] = 0.f;
    }

  // per group: area 0, area 1 (by step parity) and a third that swallows padded lanes' stores
  // partial sums travel as 32-bit words for 16-bit storage types, as 64-bit words for fp32
  typedef typename std::conditional<sizeof(T) == 2, Part32, Part64>::type PT;
  typedef typename PT::Word IW;
  IW* const inbox = reinterpret_cast<IW*>(a.ll) + (size_t)grp * 3 * INW;

  // operands of one step.  s_t is not among them: it is the s_(t-1) of the step before (kept in
  // registers, `sn` below), so only the first step loads it
  // recompute mode: h_(t-1) of the whole head (TR rows x D) goes from the stored states to LDS in pieces of HC
  // consecutive elements of one row (a power of two, at most 8: a piece never straddles an 8-element group of
  // the fragment order), NCHK pieces per thread (the last may fall beyond the end: loads return 0, no write)
  constexpr int HPT = D * TR / NT;  // elements per thread, rounded down
  constexpr int HC = HPT >= 8 ? 8 : HPT >= 4 ? 4 : HPT >= 2 ? 2 : 1;
  constexpr int HPIECES = D * TR / HC, NCHK = (HPIECES + NT - 1) / NT;
  constexpr int HCW = NDW<T, HC>::value;
  constexpr bool HSB = NDW<T, HC>::SUB;
  int h_row[NCHK], h_k0[NCHK];
  unsigned hs_v[NCHK], h0_v[NCHK];
  bool h_in[NCHK];
#pragma unroll
  for (int j = 0; j < NCHK; ++j) {
    const int piece = tid + j * NT;
    h_in[j] = piece < HPIECES;
    // (consecutive threads take the TR rows of one piece position: in fragment order a row's pieces lie 256 bytes
    // apart, i.e. in the same banks, and a wave that writes 64 pieces of one row does so in 32 passes)
    h_row[j] = piece % TR; h_k0[j] = (piece / TR) * HC;
    const bool ok = h_in[j] && bt * TR + h_row[j] < B;
    hs_v[j] = ok ? ((unsigned)(bt * TR + h_row[j]) * Tn * ND + n * D + h_k0[j]) * ES : kInvalidOff;
    h0_v[j] = ok ? ((unsigned)(bt * TR + h_row[j]) * ND + n * D + h_k0[j]) * ES : kInvalidOff;
  }
  struct Pre {
    Dw<NWC> cache[UTW]; Dw<ND_> sp[UTW][S], dso[UTW][S];
    Dw<ND_> wx[RC ? UTW : 1][RC ? GW : 1]; Dw<HCW> hrow[NCHK];  // recompute mode: Wx_t, pieces of h_(t-1)
  };
  // operands are fetched PD steps ahead into a ring of PD + 1 register sets: a head that
  // exchanges nothing (KW = 1) has steps shorter than a fetch from HBM takes.  Recompute mode: two steps
  // ahead, because the rebuild of the gates of step t-1 uses the operands of step t-1 during step t
#ifdef FRNN_PD
  constexpr int PD = RC ? 2 : KW == 1 ? FRNN_PD : 1;
#else
  constexpr int PD = RC ? 2 : KW > 1 || WAVES >= 8 || PW ? 1 : 3;  // measured: with 8 waves and more, other waves hide the fetch
#endif
  Pre pre[PD + 1];
  auto load_pre = [&](Pre& p, int t) __attribute__((always_inline)) {
    const bool first = t == 0;
    const rsrc_t rPrev = first ? rS0 : rSt;
    if constexpr (RC) {
#pragma unroll
      for (int j = 0; j < NCHK; ++j) {
        if constexpr (HSB) p.hrow[j] = buf_load<1, true>(rPrev, first ? h0_v[j] : hs_v[j], first ? 0u : (unsigned)(t - 1) * ND * ES);
        else p.hrow[j] = buf_load_wide<HCW>(rPrev, first ? h0_v[j] : hs_v[j], first ? 0u : (unsigned)(t - 1) * ND * ES);
      }
    }
#pragma unroll
    for (int u = 0; u < UTW; ++u) {
      if constexpr (RC) {
#pragma unroll
        for (int g = 0; g < GW; ++g) p.wx[u][g] = buf_load<ND_, SB>(rWx, wx_v[u], ((unsigned)t * GW + g) * ND * ES);
      }
      if constexpr (NC > 0 && !RC)
        p.cache[u] = buf_load_wide<NWC>(rCa, ca_v[u], (((unsigned)t * N + n) * (D / 16)) * Bpad * 16 * NCP * ES);
#pragma unroll
      for (int k = 0; k < S; ++k) {
        const unsigned so = ((unsigned)k * BS * Tn + t) * ND * ES;
        p.dso[u][k] = buf_load<ND_, SB>(rDs, st_v[u], so);
        if (CXU && k == CXS) continue;
        p.sp[u][k] = buf_load<ND_, SB>(rPrev, first ? s0_v[u] : st_v[u], first ? (unsigned)k * BS * ND * ES : so - ND * ES);
      }
    }
  };
#pragma unroll
  for (int i = 0; i < PD; ++i) load_pre(pre[i], Tn - 1 - i > 0 ? Tn - 1 - i : 0);
  Dw<ND_> sn[UTW][S];
#pragma unroll
  for (int u = 0; u < UTW; ++u)
#pragma unroll
    for (int k = 0; k < S; ++k) sn[u][k] = buf_load<ND_, SB>(rSt, st_v[u], ((unsigned)k * BS * Tn + (Tn - 1)) * ND * ES);
  // exchange stores may stay in the L2 of the XCD once the group is known to share one
  if (KW > 1 && w == 0) {
    const int r = (a.xcd && !a.cut) ? xcd_handshake<KW>(a.xcd + (size_t)grp * 32, slice, lane, a.status, a.spin_limit) : 0;
    if (lane == 0) near_word = r;
  }
  __syncthreads();
  const int near_i = KW > 1 ? __builtin_amdgcn_readfirstlane(near_word) : 0;  // 1: stores stay in the XCD's L2, -1: wait ran out
  u64 near_m;  // lane mask for ll_store_sel: all ones or zero, in scalar registers
  asm("s_cmp_gt_i32 %1, 0\n\ts_cselect_b64 %0, -1, 0" : "=s"(near_m) : "s"(near_i) : "scc");

#ifdef FRNN_TRACE
  long long tr[5] = {0, 0, 0, 0, 0};
  const long long tr_begin = clock64();
#endif
  // recompute mode: the rebuilt gates of the step whose adjoint comes next
  float gc[RC ? UTW : 1][NCA][E];
  // h_(tau-1), this thread's piece (from the operands of step tau), to the LDS buffer of step tau
  auto stage_h = [&](const Pre& p, int tau) __attribute__((always_inline)) {
    T* const hb = (tau & 1) ? hb1 : hb0;
#pragma unroll
    for (int j = 0; j < NCHK; ++j) {
      float v[HC];
      unpack<HC>(p.hrow[j], v, (T*)0);
      if (NCHK * NT == HPIECES || h_in[j]) {
        if constexpr (HC >= 4) {
#pragma unroll
          for (int i = 0; i < HC; i += 4) lds_write<4>(hb, h_row[j], h_k0[j] + i, v + i);
        } else {
          lds_write<HC>(hb, h_row[j], h_k0[j], v);
        }
      }
    }
  };
  // the gates of step tau from its operands and h_(tau-1) in LDS (staged before the last barrier), in two
  // halves: the forward product R h_(tau-1) of the own units, then the gate math
  auto rebuild_fetch = [&](int tau, Frag (&hq)[KSF]) __attribute__((always_inline)) {
    const Frag* hf = reinterpret_cast<const Frag*>((tau & 1) ? hb1 : hb0) + lane;
#pragma unroll
    for (int ks = 0; ks < KSF; ++ks) hq[ks] = hf[ks * 64];
  };
  auto rebuild_product = [&](const Frag (&hq)[KSF], f32x4 (&acc)[UTW][GR]) __attribute__((always_inline)) {
#pragma unroll
    for (int ks = 0; ks < KSF; ++ks)
#pragma unroll
      for (int u = 0; u < UTW; ++u)
#pragma unroll
        for (int g = 0; g < GR; ++g)
          acc[u][g] = X::mfma(rfw[u][g][ks], hq[ks], ks == 0 ? (BIAS_C ? biasc[u][g] : f32x4{0.f, 0.f, 0.f, 0.f}) : acc[u][g]);
  };
  auto rebuild_math = [&](const Pre& p, const f32x4 (&acc)[UTW][GR]) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < UTW; ++u) {
      float ryv[GR][E], wxv[GW][E], spv[S][E];
#pragma unroll
      for (int g = 0; g < GR; ++g) {
        own_elems<TR>(acc[u][g], ryv[g]);
        if constexpr (!BIAS_C) {
#pragma unroll
          for (int e = 0; e < E; ++e) ryv[g][e] += bown[u][g][e];
        }
      }
#pragma unroll
      for (int g = 0; g < GW; ++g) unpack<E>(p.wx[u][g], wxv[g], (T*)0);
#pragma unroll
      for (int k = 0; k < S; ++k) unpack<E>(p.sp[u][k], spv[k], (T*)0);
#pragma unroll
      for (int e = 0; e < E; ++e) {
        float ry[GR], wx[GW], sv[S], cc[NCA];
#pragma unroll
        for (int g = 0; g < GR; ++g) ry[g] = ryv[g][e];
#pragma unroll
        for (int g = 0; g < GW; ++g) wx[g] = wxv[g][e];
#pragma unroll
        for (int k = 0; k < S; ++k) sv[k] = spv[k][e];
        CM::fwd(ry, wx, bxr[u][e], sv, cc);
#pragma unroll
        for (int c = 0; c < NC; ++c) gc[u][c][e] = cc[c];
      }
    }
    // the rebuilt gates are used in the next step only; left alone, the compiler sinks their gate math behind
    // the wait that follows, onto the chain of dependent steps
#pragma unroll
    for (int u = 0; u < UTW; ++u)
#pragma unroll
      for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int e = 0; e < E; ++e) asm volatile("" : "+v"(gc[u][c][e]) : : "memory");
  };
  auto rebuild_gates = [&](const Pre& p, int tau) __attribute__((always_inline)) {
    f32x4 acc[UTW][GR];
    Frag hq[KSF];
    rebuild_fetch(tau, hq);
    rebuild_product(hq, acc);
    rebuild_math(p, acc);
  };
  if constexpr (RC) {  // the gates of the first reverse step
    stage_h(pre[0], Tn - 1);
    __syncthreads();
    rebuild_gates(pre[0], Tn - 1);
  }

  bool dead = near_i < 0, fail = false;
  // one reverse step: consumes `pc` (operands of step t), prefetches those of step t-1 into `pn`.
  // CUT (a std::bool_constant): truncated backpropagation, the step ends with the pointwise carry;
  // it is a compile-time variant of the step so that the full step carries no trace of it
  // (a run-time early exit cost 8 % at D = 128)
  // Recompute mode: `pm` holds the operands of step t-1, whose gates are rebuilt during this step.
  auto step = [&](auto CUT, const int t, Pre& pc, Pre& pm, Pre& pn) __attribute__((always_inline)) {
    constexpr bool cut = decltype(CUT)::value;
    T* const gb = (t & 1) ? gbuf1 : gbuf0;
    FRNN_STAMP(c0);
    // (readfirstlane: the compiler otherwise forms max(t - PD, 0) with a saturating VALU subtract
    // and then wraps a buffer load that uses it as a scalar offset into a waterfall loop)
    if constexpr (!(PW && !cut)) { if (DSP == 1 || hf == 0) load_pre(pn, __builtin_amdgcn_readfirstlane(t >= PD ? t - PD : 0)); }
    // dWx_t (and the GRU's g-gate cotangent).  With an exchange the stores are issued after the
    // partial sums are sent, where they fill the wait for the other workgroups instead of delaying
    // the barrier (a vector memory instruction costs ~30 cycles to issue)
    constexpr bool DW_LATE = KW > 1 && GW > 1;  // (a single store, Elman, measured no better behind the send)
    Dw<ND_> dwp[UTW][GW], dxp[UTW];
    auto store_dw = [&](int u) __attribute__((always_inline)) {
#pragma unroll
      for (int g = 0; g < GW; ++g) buf_store<ND_, SB>(dwp[u][g], rDw, wx_v[u], ((unsigned)t * GW + g) * ND * ES);
      if (F == FRNN_GRU) buf_store<ND_, SB>(dxp[u], rDx, st_v[u], (unsigned)t * ND * ES);
    };
    if (DSP == 1 || hf == 0) {  // (wave-uniform: the second wave of a pair owns no element)
#pragma unroll
    for (int u = 0; u < UTW; ++u) {
      float cv[NCA][E], spv[S][E], snv[S][E], dsov[S][E];
      if constexpr (NC > 0 && !RC) cache_unpack<T, NCA, E>(pc.cache[u], cv);
      if constexpr (NC > 0 && RC) {
#pragma unroll
        for (int c = 0; c < NC; ++c)
#pragma unroll
          for (int e = 0; e < E; ++e) cv[c][e] = gc[u][c][e];
      }
#pragma unroll
      for (int k = 0; k < S; ++k) {
        unpack<E>(sn[u][k], snv[k], (T*)0); unpack<E>(pc.dso[u][k], dsov[k], (T*)0);
        if (CXU && k == CXS) {  // (from the cache line; packed again, exactly, for the next step)
#pragma unroll
          for (int e = 0; e < E; ++e) spv[k][e] = cv[NC][e];
          sn[u][k] = pack<E>(cv[NC], (T*)0);
          continue;
        }
        unpack<E>(pc.sp[u][k], spv[k], (T*)0);
        sn[u][k] = pc.sp[u][k];  // s_(t-1) is the s_t of the next step
      }
      float dgr[GR][E], dgw[GW][E];
#pragma unroll
      for (int e = 0; e < E; ++e) {
        float cc[NCA], sp[S], sn[S], dso[S], gr[GR], gw[GW], gb_[GT];
#pragma unroll
        for (int c = 0; c < NC; ++c) cc[c] = cv[c][e];
#pragma unroll
        for (int k = 0; k < S; ++k) { sp[k] = spv[k][e]; sn[k] = snv[k][e]; dso[k] = dsov[k][e]; }
        ds[u][e][0] = clamp_if(ds[u][e][0], a.g_clip);
        CM::bwd(cc, sp, sn, dso, ds[u][e], gr, gw, gb_);
        // padded batch rows contribute nothing (selects, not branches)
#pragma unroll
        for (int g = 0; g < GR; ++g) dgr[g][e] = bvalid ? gr[g] : 0.f;
#pragma unroll
        for (int g = 0; g < GW; ++g) dgw[g][e] = bvalid ? gw[g] : 0.f;
#pragma unroll
        for (int g = 0; g < GT; ++g) dbacc[u][e][g] += bvalid ? gb_[g] : 0.f;
#pragma unroll
        for (int k = 0; k < S; ++k) ds[u][e][k] = bvalid ? ds[u][e][k] : 0.f;
      }
      if constexpr (DW_LATE && !cut) {
#pragma unroll
        for (int g = 0; g < GW; ++g) dwp[u][g] = pack<E>(dgw[g], (T*)0);
        if (F == FRNN_GRU) dxp[u] = pack<E>(dgr[0], (T*)0);
      } else if constexpr (PST && !cut) {  // to LDS as they lie in memory; the producer wave stores them behind this step's barrier
        T* const db = dbuf + ((Tn - 1 - t) & 1) * DB;
#pragma unroll
        for (int g = 0; g < GW; ++g)
          *reinterpret_cast<unsigned short*>(db + (g * TR + brow) * DBR + ub[u] + esub) = (unsigned short)pack<E>(dgw[g], (T*)0).v[0];
        if (F == FRNN_GRU)
          *reinterpret_cast<unsigned short*>(db + DB_W + brow * DBR + ub[u] + esub) = (unsigned short)pack<E>(dgr[0], (T*)0).v[0];
      } else {
#pragma unroll
        for (int g = 0; g < GW; ++g)
          buf_store<ND_, SB>(pack<E>(dgw[g], (T*)0), rDw, wx_v[u], ((unsigned)t * GW + g) * ND * ES);
        if (F == FRNN_GRU) buf_store<ND_, SB>(pack<E>(dgr[0], (T*)0), rDx, st_v[u], (unsigned)t * ND * ES);
      }
      if constexpr (!cut) {
#pragma unroll
        for (int g = 0; g < GR; ++g) {
          if constexpr (M44) reinterpret_cast<float*>(gb)[lds_index4(brow, g * DL + (ub[u] + esub - slice * DL))] = dgr[g][0];
          else lds_write<E>(gb, brow, g * DL + (ub[u] + esub - slice * DL), dgr[g]);
        }
      }
    }
    }
    if constexpr (RC) {
      if (t > 0) stage_h(pm, t - 1);  // uniform
    }
    if constexpr (cut) {
      if constexpr (RC) {
        if (t > 0) { lds_barrier(); rebuild_gates(pm, t - 1); }
      }
      return;
    }
    FRNN_STAMP(c1);
    // the barrier also spreads a failed wait of the previous step to the whole workgroup
    if (barrier_or(fail, dead_flag)) { dead = true; return; }
    FRNN_STAMP(c2);
    if constexpr (PW) {
      // the operands of step t-1 from the producer wave's buffer (behind this step's barrier; used in the next step)
      static_assert(E == 1 && ND_ == 1 && PD == 1, "4-row tiles: one element per lane and tile, one step ahead");
      const T* const pb = pbuf + ((Tn - t) & 1) * PB;
#pragma unroll
      for (int u = 0; u < UTW; ++u) {
        const int el = ((w * UTW + u) * TR + brow) * 16 + esub;
        if constexpr (NC > 0) {
          const unsigned* const pc_ = reinterpret_cast<const unsigned*>(pb) + el * NWC;
#pragma unroll
          for (int i = 0; i < NWC; ++i) pn.cache[u].v[i] = pc_[i];
        }
#pragma unroll
        for (int k = 0; k < S; ++k) {
          pn.sp[u][k].v[0] = reinterpret_cast<const unsigned short*>(pb + PB_CA)[k * UT_WG * TR * 16 + el];
          pn.dso[u][k].v[0] = reinterpret_cast<const unsigned short*>(pb + PB_CA + PB_ST)[k * UT_WG * TR * 16 + el];
        }
      }
    }

    // one accumulator per tile: splitting a lone chain over several accumulators (as the forward
    // kernel does) measured 3-8 % slower here, before and after the barrier was made LDS-only
    constexpr int NACC = 1;
    // With 3 and more workgroups per head the products that other workgroups wait for come first
    // and are sent at once; the product for the own tiles follows while those words travel (it
    // needs all fragments still in registers: one chunk)
    constexpr bool OWN_LAST = KW >= 3 && KS == chunk_of(KS) && !M44;
    // More than 8 remote destinations (10 and more workgroups per head): their products run in groups
    // of 4 destinations (4 independent MFMA chains), each group sent as soon as it is complete, so that
    // 16 accumulator registers are live instead of 4 per destination (128 at 32 workgroups per head).
    constexpr bool GROUPED = OWN_LAST && KW - 1 > 8;
    constexpr int RI = 4;
    static_assert(!GROUPED || RLD % RI == 0, "LDS-resident destinations come in whole groups");
    static_assert(!DS16 || GROUPED, "wave pairs split the destinations of the grouped product only");
    const int hfo = DS16 ? hf * NL : 0;  // first destination of this wave (uniform)
    float p44[M44 ? NGH : 1][M44 ? UTW : 1][4];  // 4x4x1 form: partial sums of the lane's element, destination 4 (q DSP + hf) + i
    if constexpr (M44) {
      const float* gfl = reinterpret_cast<const float*>(gb) + lane;
      float ga[KDL / 16];
#pragma unroll
      for (int v = 0; v < KDL / 16; ++v) ga[v] = gfl[64 * v];
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int q = 0; q < NGH; ++q)
#pragma unroll
        for (int u = 0; u < UTW; ++u) {
          f32x4 ac[4];
#pragma unroll
          for (int v = 0; v < KDL / 16; ++v) mfma_4x4x1_bcast16(ga[v], &rtb[q][u][16 * v], ac, v == 0);
          const f32x4 sum = (ac[0] + ac[1]) + (ac[2] + ac[3]);
          // lane 4*blk + j holds (destination 4q + j, unit blk) of batch rows 0..3; after the transpose lane
          // 4*blk + b holds destinations 4q .. 4q+3 of (batch row b, unit blk): the element of this lane
          p44[q][u][0] = sum[0]; p44[q][u][1] = sum[1]; p44[q][u][2] = sum[2]; p44[q][u][3] = sum[3];
          quad_transpose(p44[q][u], lane);
        }
#pragma unroll
      for (int u = 0; u < UTW; ++u) ds[u][0][0] += p44[0][u][0];  // (the own tiles: destination 0 of the first wave)
    }
    f32x4 accp[NACC][GROUPED ? 1 : KW][UTW];
    const Frag* gf = reinterpret_cast<const Frag*>(gb) + lane;
    constexpr int KC = chunk_of(KS);
    static_assert(KS % KC == 0, "k-steps must split into whole chunks");
    Frag gq[2][KC];
#pragma unroll
    for (int k = 0; k < (M44 ? 0 : KC); ++k) gq[0][k] = gf[k * 64];
    Frag la_next[RLD > 0 ? RLD : 1][UTW];
    if constexpr (RLD > 0 && !GROUPED) {
#pragma unroll
      for (int rr = 0; rr < RLD; ++rr)
#pragma unroll
        for (int u = 0; u < UTW; ++u) la_next[rr][u] = rl[((rr * UTW + u) * KS) * 64];
    }
    // keep the reads up here: issued just in time they would expose the LDS latency once per chunk
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (GROUPED) {
      const unsigned sslot = ((unsigned)(rvalid ? (t & 1) : 2) * (unsigned)INW + lane) * (unsigned)sizeof(IW);  // byte offset of the area + lane
      auto send_group = [&](int r0, int nr, f32x4 (&ag)[RI][UTW]) __attribute__((always_inline)) {
        if (nr == RI) {  // (compile-time at every call site) four destinations with one switch of the store form
#pragma unroll
          for (int u = 0; u < UTW; ++u) {
            const void* base[RI];
            IW wv[RI][E];
#pragma unroll
            for (int rr = 0; rr < RI; ++rr) {
              const int x = (slice + hfo + r0 + rr) % KW;
              base[rr] = inbox + (size_t)(((x * NPOS + wp_u) * UTW + u) * KW + slice) * 256;
              float part[E];
              own_elems<TR>(ag[rr][u], part);
#pragma unroll
              for (int e = 0; e < E; ++e) wv[rr][e] = part_pack((PT*)0, part[e], t);
            }
            ll_store_sel4<E, 64 * (int)sizeof(IW)>(base, sslot, wv, near_m);
          }
          return;
        }
#pragma unroll
        for (int rr = 0; rr < RI; ++rr) {
          if (rr >= nr) continue;
          const int x = (slice + hfo + r0 + rr) % KW;
#pragma unroll
          for (int u = 0; u < UTW; ++u) {
            float part[E];
            own_elems<TR>(ag[rr][u], part);
            IW wv[E];
#pragma unroll
            for (int e = 0; e < E; ++e) wv[e] = part_pack((PT*)0, part[e], t);
            // (the destination's place in the area is uniform and goes into the scalar base; the lane's offset is the same for all)
            ll_store_sel<E, 64 * (int)sizeof(IW)>(inbox + (size_t)(((x * NPOS + wp_u) * UTW + u) * KW + slice) * 256, sslot, wv, near_m);
          }
        }
      };
      // destinations whose fragments are in registers
#pragma unroll
      for (int r0 = 1; r0 < KWR; r0 += RI) {
        const int nr = KWR - r0 < RI ? KWR - r0 : RI;
        f32x4 ag[RI][UTW];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
          for (int rr = 0; rr < RI; ++rr)
#pragma unroll
            for (int u = 0; u < UTW; ++u)
              if (rr < nr) ag[rr][u] = X::mfma(rtf[r0 + rr < KWR ? r0 + rr : 0][u][ks], gq[0][ks], ks == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : ag[rr][u]);
          __builtin_amdgcn_sched_barrier(0);
        }
        send_group(r0, nr, ag);
      }
      // destinations whose fragments are in LDS: those of the next (group, k-step) are requested before
      // the MFMAs of the current one
      if constexpr (RLD > 0) {
        Frag lb[2][RI][UTW];
#pragma unroll
        for (int rr = 0; rr < RI; ++rr)
#pragma unroll
          for (int u = 0; u < UTW; ++u) lb[0][rr][u] = rl[((rr * UTW + u) * KS) * 64];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int gi = 0; gi < RLD / RI; ++gi) {
          f32x4 ag[RI][UTW];
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            const int m = gi * KS + ks, mn = m + 1;
            if (mn < (RLD / RI) * KS) {
              const int gn = mn / KS, kn = mn % KS;
#pragma unroll
              for (int rr = 0; rr < RI; ++rr)
#pragma unroll
                for (int u = 0; u < UTW; ++u) lb[mn & 1][rr][u] = rl[(((gn * RI + rr) * UTW + u) * KS + kn) * 64];
              __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int rr = 0; rr < RI; ++rr)
#pragma unroll
              for (int u = 0; u < UTW; ++u)
                ag[rr][u] = X::mfma(lb[m & 1][rr][u], gq[0][ks], ks == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : ag[rr][u]);
            __builtin_amdgcn_sched_barrier(0);
          }
          send_group(KWR + gi * RI, RI, ag);
        }
      }
    }
#pragma unroll
    for (int kc = 0; kc < (GROUPED || M44 ? 0 : KS / KC); ++kc) {
      if (kc + 1 < KS / KC) {
#pragma unroll
        for (int k = 0; k < KC; ++k) gq[(kc + 1) & 1][k] = gf[((kc + 1) * KC + k) * 64];
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int k = 0; k < KC; ++k) {
        const int ks = kc * KC + k, j = ks % NACC;
        // fragments kept in LDS: those of the next k-step are requested before this one's MFMAs
        Frag la[RLD > 0 ? RLD : 1][UTW];
        if constexpr (RLD > 0) {
#pragma unroll
          for (int rr = 0; rr < RLD; ++rr)
#pragma unroll
            for (int u = 0; u < UTW; ++u) la[rr][u] = la_next[rr][u];
          if (ks + 1 < KS) {
#pragma unroll
            for (int rr = 0; rr < RLD; ++rr)
#pragma unroll
              for (int u = 0; u < UTW; ++u) la_next[rr][u] = rl[((rr * UTW + u) * KS + ks + 1) * 64];
          }
          __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int r = OWN_LAST ? 1 : 0; r < KW; ++r)
#pragma unroll
          for (int u = 0; u < UTW; ++u)
            accp[j][r][u] = X::mfma(r < KWR ? rtf[r < KWR ? r : 0][u][ks] : la[r < KWR ? 0 : r - KWR][u], gq[kc & 1][k],
                                    ks < NACC ? f32x4{0.f, 0.f, 0.f, 0.f} : accp[j][r][u]);
        if (j == NACC - 1) __builtin_amdgcn_sched_barrier(0);
      }
    }
    static_assert(NACC == 1, "one accumulator per tile");
    f32x4 acc[GROUPED ? 1 : KW][UTW];
#pragma unroll
    for (int r = OWN_LAST ? 1 : 0; r < (GROUPED || M44 ? 0 : KW); ++r)
#pragma unroll
      for (int u = 0; u < UTW; ++u) acc[r][u] = accp[0][r][u];
    if constexpr (!OWN_LAST && !M44) {
#pragma unroll
      for (int u = 0; u < UTW; ++u) {
        float own[E];
        own_elems<TR>(acc[0][u], own);
#pragma unroll
        for (int e = 0; e < E; ++e) ds[u][e][0] += own[e];
      }
    }

#ifdef FRNN_TRACE
    { float sink = 0.f;
#pragma unroll
      for (int u = 0; u < UTW; ++u) sink += ds[u][0][0];
      asm volatile("" ::"v"(sink)); }
#endif
    FRNN_STAMP(c3);
    if constexpr (KW > 1) {
      // send: partial sums of the tiles owned by workgroup (slice + r) % KW, same wave position
      const unsigned sslot = ((unsigned)(rvalid ? (t & 1) : 2) * (unsigned)INW + lane) * (unsigned)sizeof(IW);  // byte offset of the area + lane
      if constexpr (DSP > 1 && M44) {  // this wave's destination groups (4x4x1 form)
#pragma unroll
        for (int q = 0; q < NGH; ++q)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int r = 4 * (q * DSP + hf) + j;
            if (r < 1 || r >= KW) continue;  // (uniform)
            const int x = (slice + r) % KW;
#pragma unroll
            for (int u = 0; u < UTW; ++u) {
              IW wv[E];
              wv[0] = part_pack((PT*)0, p44[q][u][j], t);
              ll_store_sel<E, 64 * (int)sizeof(IW)>(inbox + (size_t)(((x * NPOS + wp_u) * UTW + u) * KW + slice) * 256, sslot, wv, near_m);
            }
          }
      }
#pragma unroll
      for (int r = 1; r < (GROUPED || DSP > 1 ? 0 : KW); ++r) {
        const int x = (slice + r) % KW;
#pragma unroll
        for (int u = 0; u < UTW; ++u) {
          float part[E];
          if constexpr (M44) part[0] = p44[r >> 2][u][r & 3];
          else own_elems<TR>(acc[r][u], part);
          IW wv[E];
#pragma unroll
          for (int e = 0; e < E; ++e) wv[e] = part_pack((PT*)0, part[e], t);
          // (the destination's place in the area is uniform and goes into the scalar base; the lane's offset is the same for all)
            ll_store_sel<E, 64 * (int)sizeof(IW)>(inbox + (size_t)(((x * NPOS + wp_u) * UTW + u) * KW + slice) * 256, sslot, wv, near_m);
        }
      }
      if constexpr (DW_LATE) {
        if (DSP == 1 || hf == 0) {
#pragma unroll
          for (int u = 0; u < UTW; ++u) store_dw(u);
        }
      }
      if constexpr (OWN_LAST) {
        // the product for the own tiles, while the words just sent travel
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
          for (int u = 0; u < UTW; ++u)
            accp[0][0][u] = X::mfma(rtf[0][u][ks], gq[0][ks], ks == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : accp[0][0][u]);
#pragma unroll
        for (int u = 0; u < UTW; ++u) {
          float own[E];
          own_elems<TR>(accp[0][0][u], own);
          if (DS16 && hf != 0) {  // (uniform) the second wave's first destination is no tile of its own: sent like the others
            IW wv[E];
#pragma unroll
            for (int e = 0; e < E; ++e) wv[e] = part_pack((PT*)0, own[e], t);
            ll_store_sel<E, 64 * (int)sizeof(IW)>(inbox + (size_t)(((((slice + hfo) % KW) * NPOS + wp_u) * UTW + u) * KW + slice) * 256, sslot, wv, near_m);
          } else {
#pragma unroll
            for (int e = 0; e < E; ++e) ds[u][e][0] += own[e];
          }
        }
      }
      // receive: KW-1 partial sums of the own tiles, PSRC sources at a time
      const IW* const mine = inbox + (size_t)(t & 1) * INW + ((size_t)(slice * NPOS + wp) * UTW) * KW * 256 + lane;
      if constexpr (RSP) {
        const int rbeg = 1 + hf * SRC_W;  // (uniform) this wave's sources: rbeg .. rbeg + SRC_W - 1, below KW
        float rs[UTW][E];
#pragma unroll
        for (int u = 0; u < UTW; ++u)
#pragma unroll
          for (int e = 0; e < E; ++e) rs[u][e] = 0.f;
#pragma unroll
        for (int k0 = 0; k0 < SRC_W; k0 += PSRC_W) {
          constexpr int NWR = PSRC_W * UTW * E;
          int off[NWR]; bool need[NWR]; IW v[NWR];
#pragma unroll
          for (int rr = 0; rr < PSRC_W; ++rr) {
            const bool in = k0 + rr < SRC_W && rbeg + k0 + rr < KW;
            const int src = (slice + (in ? rbeg + k0 + rr : 1)) % KW;
#pragma unroll
            for (int u = 0; u < UTW; ++u)
#pragma unroll
              for (int e = 0; e < E; ++e) {
                off[(rr * UTW + u) * E + e] = (u * KW + src) * 256 + e * 64;
                need[(rr * UTW + u) * E + e] = rvalid && in;
              }
          }
          if (!fail) fail = poll_words_staggered<PT, NWR>(mine, off, need, t, v, a.status, a.spin_limit, k0 == 0 ? a.poll_delay : 0);
#pragma unroll
          for (int rr = 0; rr < PSRC_W; ++rr) {
            const bool in = k0 + rr < SRC_W && rbeg + k0 + rr < KW;
#pragma unroll
            for (int u = 0; u < UTW; ++u)
#pragma unroll
              for (int e = 0; e < E; ++e) rs[u][e] += in ? part_value((PT*)0, v[(rr * UTW + u) * E + e]) : 0.f;
          }
        }
        // (the buffer is free again before the next write: the barrier of the next step lies in between)
        if (hf != 0) {
#pragma unroll
          for (int u = 0; u < UTW; ++u)
#pragma unroll
            for (int e = 0; e < E; ++e) rsum[(((wp_u * (DSP - 1) + hf - 1) * UTW + u) * E + e) * 64 + lane] = rs[u][e];
        }
        lds_barrier();
        if (hf == 0) {
#pragma unroll
          for (int u = 0; u < UTW; ++u)
#pragma unroll
            for (int e = 0; e < E; ++e) {
              float sum = rs[u][e];
#pragma unroll
              for (int i = 0; i < DSP - 1; ++i) sum += rsum[(((wp_u * (DSP - 1) + i) * UTW + u) * E + e) * 64 + lane];
              ds[u][e][0] += sum;
            }
        }
      } else if (DSP == 1 || hf == 0) {
#pragma unroll
      for (int r0 = 1; r0 < KW; r0 += PSRC) {
        constexpr int NWR = PSRC * UTW * E;
        int off[NWR]; bool need[NWR]; IW v[NWR];
#pragma unroll
        for (int rr = 0; rr < PSRC; ++rr) {
          const int src = (slice + (r0 + rr < KW ? r0 + rr : 1)) % KW;
#pragma unroll
          for (int u = 0; u < UTW; ++u)
#pragma unroll
            for (int e = 0; e < E; ++e) {
              off[(rr * UTW + u) * E + e] = (u * KW + src) * 256 + e * 64;
              need[(rr * UTW + u) * E + e] = bvalid && (r0 + rr < KW);
            }
        }
        if constexpr (RC) {
          // recompute mode: the gates of step t-1 are rebuilt while the partial sums of step t travel.  The
          // first probe is sent early (behind the LDS reads of the rebuild, which stand in for the delay of the
          // cached path: a probe that reaches memory before the words costs a second round trip of ~1200
          // cycles) and the forward product and the gate math run behind its round trip
          static_assert(ROUNDS == 1, "recompute mode: one round of polling");
          f32x4 racc[UTW][GR];
          Frag rhq[KSF];
          if (t > 0) rebuild_fetch(t - 1, rhq);
          __builtin_amdgcn_sched_barrier(0);
          for (int i = 0; i < a.poll_delay; ++i) __builtin_amdgcn_s_sleep(1);
          IW pv[NWR];
          poll_issue<NWR>(mine, off, pv);
          __builtin_amdgcn_sched_barrier(0);
          if (t > 0) { rebuild_product(rhq, racc); rebuild_math(pm, racc); }
          if (!fail) fail = poll_finish<PT, NWR>(mine, off, need, t, pv, v, a.status, a.spin_limit);
        } else {
          if (!fail) fail = poll_words_staggered<PT, NWR>(mine, off, need, t, v, a.status, a.spin_limit, r0 == 1 ? a.poll_delay : 0);
        }
#pragma unroll
        for (int rr = 0; rr < PSRC; ++rr)
          if (r0 + rr < KW) {
#pragma unroll
            for (int u = 0; u < UTW; ++u)
#pragma unroll
              for (int e = 0; e < E; ++e) ds[u][e][0] += part_value((PT*)0, v[(rr * UTW + u) * E + e]);
          }
      }
      }
    }
    if constexpr (RC && KW == 1) {
      if (t > 0) rebuild_gates(pm, t - 1);
    }
#ifdef FRNN_TRACE
    FRNN_STAMP(c4);
    tr[0] += c1 - c0; tr[1] += c2 - c1; tr[2] += c3 - c2; tr[3] += c4 - c3;
#endif
  };

  // the time loop, unrolled over the ring: step t - j consumes set j and refills the set that the
  // step before it consumed
  int t = Tn - 1;
  if constexpr (RC) {
    // ring of 3 sets: step t consumes set j (its own operands) and set j+1 (those of step t-1, for the
    // rebuild) and refills set j+2 with the operands of step t-2
    auto run = [&](auto CUT) __attribute__((always_inline)) {
      for (; t >= 2 && !dead; t -= 3) {
        step(CUT, t, pre[0], pre[1], pre[2]);
        if (dead) break;
        step(CUT, t - 1, pre[1], pre[2], pre[0]);
        if (dead) break;
        step(CUT, t - 2, pre[2], pre[0], pre[1]);
      }
      if (!dead && t >= 0) {
        step(CUT, t, pre[0], pre[1], pre[2]);
        if (!dead && t >= 1) step(CUT, t - 1, pre[1], pre[2], pre[0]);
      }
    };
    if (a.cut) run(std::true_type{}); else run(std::false_type{});
  } else if (a.cut) {
    for (; t >= PD; t -= PD + 1) {
#pragma unroll
      for (int j = 0; j <= PD; ++j) step(std::true_type{}, t - j, pre[j], pre[j], pre[(j + PD) % (PD + 1)]);
    }
#pragma unroll
    for (int j = 0; j < PD; ++j)
      if (t - j >= 0) step(std::true_type{}, t - j, pre[j], pre[j], pre[(j + PD) % (PD + 1)]);
  } else if constexpr (PD == 1) {
    // (written out: in the general form below the register allocation of the largest kernels,
    // which sit at the 256-register limit, comes out with spills)
    for (; t >= 1 && !dead; t -= 2) {
      step(std::false_type{}, t, pre[0], pre[0], pre[1]);
      if (dead) break;
      step(std::false_type{}, t - 1, pre[1], pre[1], pre[0]);
    }
    if (!dead && t == 0) step(std::false_type{}, 0, pre[0], pre[0], pre[1]);
  } else {
    for (; t >= PD && !dead; t -= PD + 1) {
#pragma unroll
      for (int j = 0; j <= PD; ++j) {
        step(std::false_type{}, t - j, pre[j], pre[j], pre[(j + PD) % (PD + 1)]);
        if (dead) break;
      }
    }
#pragma unroll
    for (int j = 0; j < PD; ++j)
      if (!dead && t - j >= 0) step(std::false_type{}, t - j, pre[j], pre[j], pre[(j + PD) % (PD + 1)]);
  }
  if (!dead && barrier_or(fail, dead_flag)) dead = true;
#ifdef FRNN_TRACE
  if (lane == 0 && a.trace) {
    long long* o = a.trace + ((size_t)blockIdx.x * WAVES + w) * 8;
    o[0] = tr[0]; o[1] = tr[1]; o[2] = tr[2]; o[3] = tr[3]; o[4] = clock64() - tr_begin; o[5] = tr[4];
  }
#endif

  if (dead) {
    if (tid == 0) __hip_atomic_store(a.status, (int)STATUS_WAIT_EXPIRED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int u = 0; u < UTW; ++u)
#pragma unroll
      for (int e = 0; e < E; ++e)
#pragma unroll
        for (int k = 0; k < S; ++k) ds[u][e][k] = __uint_as_float(0x7fc00000u);
  }

  // ---- cotangent of the initial state, bias partial sums ----------------------------------
  const rsrc_t rD0 = make_rsrc(a.ds0, ((size_t)(S - 1) * BS + B) * ND * ES);
#pragma unroll
  for (int u = 0; u < UTW; ++u) {
#pragma unroll
    for (int k = 0; k < S; ++k) {
      float v[E];
#pragma unroll
      for (int e = 0; e < E; ++e) v[e] = ds[u][e][k];
      buf_store<ND_, SB>(pack<E>(v, (T*)0), rD0, s0_v[u], (unsigned)k * BS * ND * ES);
    }
#pragma unroll
    for (int g = 0; g < GT; ++g)
#pragma unroll
      for (int e = 0; e < E; ++e) {
        float v = dead ? __uint_as_float(0x7fc00000u) : dbacc[u][e][g];
        v += __shfl_xor(v, 1); v += __shfl_xor(v, 2);
        if (TR >= 8) v += __shfl_xor(v, 4);
        if (TR == 16) v += __shfl_xor(v, 8);
        if (brow == 0 && (DSP == 1 || hf == 0)) a.dbp[(((size_t)bt * GT + g) * N + n) * D + ub[u] + esub + e] = v;
      }
  }
}

}  // namespace frnn
