// extern "C" surface of libflashrnn_hip.so: argument validation (host only, before any launch),
// workspace carving, launch sequencing.  No device allocation, no hidden streams, no
// device-wide synchronisation.
#include <stdarg.h>
#include <stddef.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>

#include "frnn_alt.h"
#include "frnn_fused_bwd.h"
#include "frnn_fused_fwd.h"
#include "frnn_grad.h"
#include "frnn_launch.h"
#include "frnn_mailbox.h"

namespace frnn {

static thread_local char g_err[512] = "";
static int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
static int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}
static int hip_fail(int e, const char* what) {
  if (e > 0) snprintf(g_err, sizeof(g_err), "%s: %s", what, hipGetErrorString((hipError_t)e));
  else if (e == FRNN_E_UNSUPPORTED) snprintf(g_err, sizeof(g_err), "%s: tiling not compiled in", what);
  return e;
}

// ---- optional per-launch timing with HIP events on the caller's stream ---------------------------
// Off by default.  When on, every kernel launch (or launch loop) of a call is bracketed by two
// events; frnn_profile_ms() waits for them.  Meant for benchmarks: one thread, one stream.
struct ProfRec { const char* name; hipEvent_t a, b; };
static const int kProfMax = 64;  // ring: the most recent kProfMax launches are kept
static ProfRec g_prof[kProfMax];
static long g_prof_n = 0;
static int g_prof_on = 0, g_prof_events = 0;
static void prof_begin(const char* name, hipStream_t st) {
  if (!g_prof_on) return;
  const int i = (int)(g_prof_n % kProfMax);
  if (g_prof_events <= i) {
    if (hipEventCreate(&g_prof[i].a) != hipSuccess || hipEventCreate(&g_prof[i].b) != hipSuccess) { g_prof_on = 0; return; }
    g_prof_events = i + 1;
  }
  g_prof[i].name = name;
  hipEventRecord(g_prof[i].a, st);
}
static void prof_end(hipStream_t st) {
  if (!g_prof_on) return;
  hipEventRecord(g_prof[(int)(g_prof_n % kProfMax)].b, st);
  ++g_prof_n;
}
static int prof_slot(int i) {  // i-th oldest entry still held -> ring slot, or -1
  const long held = g_prof_n < kProfMax ? g_prof_n : kProfMax;
  if (i < 0 || i >= held) return -1;
  return (int)((g_prof_n - held + i) % kProfMax);
}

// ---- plan table -------------------------------------------------------------------------------
#define FRNN_ROW(Dv, VAR, W, U, K, MTR) {Dv, VAR, W, U, K, MTR},
static const Plan kFwd4B[] = {FRNN_PLANS_GR4_BF16(FRNN_ROW)};
static const Plan kFwd4F[] = {FRNN_PLANS_GR4_F32(FRNN_ROW)};
static const Plan kFwdSB[] = {FRNN_PLANS_SLSTM_BF16(FRNN_ROW)};
static const Plan kFwd3B[] = {FRNN_PLANS_GR3_BF16(FRNN_ROW)};
static const Plan kFwd3F[] = {FRNN_PLANS_GR3_F32(FRNN_ROW)};
static const Plan kFwd1B[] = {FRNN_PLANS_GR1_BF16(FRNN_ROW)};
static const Plan kFwd1F[] = {FRNN_PLANS_GR1_F32(FRNN_ROW)};
static const Plan kBwd4B[] = {FRNN_BWD_PLANS_GR4_BF16(FRNN_ROW)};
static const Plan kBwdSB[] = {FRNN_BWD_PLANS_SLSTM_BF16(FRNN_ROW)};
static const Plan kBwd4F[] = {FRNN_BWD_PLANS_GR4_F32(FRNN_ROW)};
static const Plan kBwdSF[] = {FRNN_BWD_PLANS_SLSTM_F32(FRNN_ROW)};
static const Plan kBwd3B[] = {FRNN_BWD_PLANS_GR3_BF16(FRNN_ROW)};
static const Plan kBwd3F[] = {FRNN_BWD_PLANS_GR3_F32(FRNN_ROW)};
static const Plan kBwd1B[] = {FRNN_BWD_PLANS_GR1_BF16(FRNN_ROW)};
static const Plan kBwd1F[] = {FRNN_BWD_PLANS_GR1_F32(FRNN_ROW)};
static const Plan kRc4B[] = {FRNN_BWD_RC_PLANS_GR4_BF16(FRNN_ROW)};
static const Plan kRcSB[] = {FRNN_BWD_RC_PLANS_SLSTM_BF16(FRNN_ROW)};
static const Plan kRc4F[] = {FRNN_BWD_RC_PLANS_GR4_F32(FRNN_ROW)};
static const Plan kRc3B[] = {FRNN_BWD_RC_PLANS_GR3_BF16(FRNN_ROW)};
static const Plan kRc3F[] = {FRNN_BWD_RC_PLANS_GR3_F32(FRNN_ROW)};
#undef FRNN_ROW

bool find_plan(int function, int dtype, int D, int variant, int backward, Plan* out) {
  const int GR = cell_dims(function).GR;
  const Plan* tab = nullptr;
  size_t n = 0;
#define PICK(T) { tab = T; n = sizeof(T) / sizeof(Plan); }
  if (!backward) {
    if (GR == 4) { if (dtype == FRNN_F32) PICK(kFwd4F) else if (function == FRNN_SLSTM) PICK(kFwdSB) else PICK(kFwd4B) }
    else if (GR == 3) { if (dtype != FRNN_F32) PICK(kFwd3B) else PICK(kFwd3F) }
    else { if (dtype != FRNN_F32) PICK(kFwd1B) else PICK(kFwd1F) }
  } else if (backward == 1) {
    if (GR == 4) {
      if (dtype == FRNN_F32) { if (function == FRNN_SLSTM) PICK(kBwdSF) else PICK(kBwd4F) }
      else if (function == FRNN_SLSTM) PICK(kBwdSB) else PICK(kBwd4B)
    }
    else if (GR == 3) { if (dtype != FRNN_F32) PICK(kBwd3B) else PICK(kBwd3F) }
    else { if (dtype != FRNN_F32) PICK(kBwd1B) else PICK(kBwd1F) }
  } else {  // reverse scan in recompute mode
    if (GR == 4) { if (dtype == FRNN_F32) PICK(kRc4F) else if (function == FRNN_SLSTM) PICK(kRcSB) else PICK(kRc4B) }
    else if (GR == 3) { if (dtype != FRNN_F32) PICK(kRc3B) else PICK(kRc3F) }
    else return false;
  }
#undef PICK
  const Plan* dflt = nullptr;
  for (size_t i = 0; i < n; ++i) {
    if (tab[i].D != D) continue;
    if (tab[i].variant == variant) { *out = tab[i]; out->recompute = backward == 2; return true; }
    if (tab[i].variant == 0) dflt = &tab[i];
  }
  if (dflt) { *out = *dflt; out->recompute = backward == 2; return true; }
  return false;
}


static int env_int(const char* name, int dflt) {
  const char* v = getenv(name);
  return (v && *v) ? atoi(v) : dflt;
}
// Exchange stores of a group whose workgroups share an XCD stay in that XCD's L2 (workgroup scope; the kernels
// check the placement themselves, see xcd_handshake).  FRNN_AGENT_STORES=1 keeps every store at agent scope.
static bool near_stores_allowed() { return env_int("FRNN_AGENT_STORES", 0) == 0; }

// s_sleep units before the first probe of a forward step.  A probe that reaches memory before the
// data costs a whole extra round trip and adds traffic, one that comes late costs its lateness; where
// the data arrives depends on how long the other workgroups' gate math and stores take, so the best
// value differs by cell and tiling.  Measured on MI355X (bf16, T = 1024, exchange stores kept in the XCD's
// L2; a unit off costs up to 1-3 %, most curves are flat within 2 units):
//   kernels that multiply the own slice in front of the wait, 4-row tiles: lstm D=256 0, D=320 0, D=512 1, D=640 1;
//   slstm D=192, 256 0, D=640 1; gru D=256, 384, 640 1, D=768 2, D=1024 (16 workgroups) 6; elman D=512, 1024 0,
//   D=640 2, fp32 0; 8- and 16-row tiles 2-4 (flat);
//   lstm, slstm D=768 (12 workgroups) 0-1;  the others: lstm D=1024 (32 workgroups of 2 waves) 3-6.
static int fwd_poll_delay_default(int function, int dtype, const Plan& p, int tile_rows) {
  if (p.kw <= 1) return 0;
  // groups that span the device exchange through memory, at agent scope: a round trip takes several times as long as
  // one to the L2 of an XCD (lstm fp32 D=1024, forward, 1024 steps: delay 0 6.09 ms, 8 4.81, 16 4.37, 24 3.92, 32 4.00, 48 4.36)
  // (the other cells and D = 768 also best at 24, within 1 %; 40 workgroups per head, D = 640: 18 2.64 ms, 24 2.74)
  if (p.kw > kXcdWorkgroups) return p.kw <= 40 ? 18 : 24;
  const bool elman = function == FRNN_ELMAN || function == FRNN_ELMAN_CLIP;
  // kernels that multiply the workgroup's own slice in front of the wait: little is left to sleep through
  if (fwd_own_slice_first(cell_dims(function).GR, p.D, p.waves, p.utw, p.kw, tile_rows, dtype == FRNN_F32 ? 4 : 2)) {
    if (elman) return p.kw > 8 && dtype != FRNN_F32 ? 2 : 0;
    if (p.kw > 8) return p.kw >= 16 ? 6 : p.kw < 12 ? 1 : function == FRNN_GRU ? 2 : 0;
    return tile_rows >= 8 ? 2 : (function == FRNN_GRU || p.kw > 5) ? 1 : 0;
  }
  if (elman) return p.waves > 4 ? 2 : 6;
  if (p.kw == 3) return 2;
  if (p.kw == 6) return 4;
  if (p.kw == 10) return 5;
  if (p.kw >= 12) return 6;
  if (p.kw == 4 && function == FRNN_GRU) return 4;
  return 3;
}

// compute units of the current device; 256 (MI355X) if no device can be queried
static int device_cus() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int cu = 0;
    if (hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cu <= 0) cu = 256;
    cached[dev] = cu;
  }
  return cached[dev];
}

// Groups (head, batch tile) of KW > 1 workgroups that one launch may hold.  The workgroups of a group wait
// for each other, so all of them must be resident, and a group is pinned to one XCD (decode_block): what
// counts is the room of an XCD (an eighth of the compute units, one such workgroup per compute unit), not
// of the device: with KW = 12 an XCD of 32 compute units holds 2 groups, the device 16, not 256 / 12 = 21.
// Heads of more than 32 workgroups (kXcdWorkgroups) spread over the whole device: what counts is the device.
static int groups_per_launch(int kw) { return kw > kXcdWorkgroups ? device_cus() / kw : 8 * ((device_cus() / 8) / kw); }
// (such groups never share an XCD: no handshake, every exchange store at agent scope)
static bool near_stores_possible(const Plan& p) { return p.kw > 1 && p.kw <= kXcdWorkgroups; }

// The tiling of a call: the table's default for the head dim, or its small-batch alternative (variant 2) while all
// groups of the call fit one launch with 4-row tiles.  FRNN_FUSED_VARIANT picks a variant by hand.
static bool pick_plan(int function, int dtype, int B, int N, int D, int backward, Plan* p) {
  const int variant = env_int("FRNN_FUSED_VARIANT", 0);
  if (!find_plan(function, dtype, D, variant, backward, p)) return false;
  if (variant == 0) {
    Plan q;
    if (find_plan(function, dtype, D, 2, backward, &q) && q.variant == 2 && q.kw > 1 &&
        (long)N * ((B + 3) / 4) <= groups_per_launch(q.kw))
      *p = q;
  }
  return true;
}

// Batch rows per group: 4, 8 or 16.  Fewer rows per tile mean less gate math per lane and fewer
// words to poll per step (the larger costs of a step) at the price of more workgroups and copies
// of R, so the smallest tile is used for which every workgroup of the call still gets a compute
// unit of its own.  Heads that run as one workgroup (no exchange) may share a compute unit, many at a time: one
// workgroup's gate math then runs while another waits for memory, and in the 16-bit types only the 4-row kernels
// have the producer wave and its 16-byte stores.  Measured (bf16, T = 1024 unless noted, 4- against 8- against 16-row
// tiles, ms per step): LSTM B = 340 N12 D64, 1020 workgroups, 4.07 / 4.80; B = 1024 T = 256 N12 D64, 3072 workgroups, 2.52 /
// 2.83 / 2.66; N8 D96 B = 1024 T = 256, 2048 workgroups of 6 waves, 3.60 / 3.98 / 3.66; N6 D128 (8 waves) B = 256, 384
// workgroups, LSTM 3.04 / 3.51 / 5.46, GRU 2.52 / 2.51 / 4.20, Elman 1.06 / 1.14 / 1.52; B = 1024 T = 256, 1536 workgroups,
// LSTM 2.64 / 2.60 / 3.00, GRU 2.27 / 2.18 / 2.56.  So: 4-row tiles up to 16 workgroups per compute unit for up to 4 waves,
// 8 for up to 6, 4 for up to 8 (fp32, without the producer wave: 8 / 4 / 4 / 1 for 2 / 4 / 6 / more waves).
// `largest` is the tallest tile the tiling is compiled for (Plan::max_tr: taller ones would spill registers).
static int tile_rows_for(int B, int N, int kw, int waves, int largest, int dtype) {
  const int forced = env_int("FRNN_TILE_ROWS", 0);
  if (forced == 4 || forced == 8 || forced == 16) return forced < largest ? forced : largest;
  const int share = dtype != FRNN_F32 ? (waves <= 4 ? 16 : waves <= 6 ? 8 : waves <= 8 ? 4 : 1)
                                      : (waves <= 2 ? 8 : waves <= 4 ? 4 : 1);
  const long room = kw > 1 ? groups_per_launch(kw) : (long)device_cus() * share;
  for (int tr = 4; tr < largest; tr *= 2)
    if ((long)N * ((B + tr - 1) / tr) <= room) return tr;
  return largest;
}

// ---- one multi-workgroup launch at a time per device ------------------------------------------------
// The workgroups of a head that spans several of them wait for each other, and a launch is sized to hold
// all its groups on the device at once.  Two such kernels that ran at the same time (calls on different
// streams) could each get a part of the device and starve each other until the bounded waits run out, so
// the library orders them: per device it remembers the stream of the last such launch, and a launch on
// another stream first waits (hipStreamWaitEvent, on the device, nothing blocks on the host) for an event
// recorded on that stream.  Calls on one stream, the normal case, pay nothing.  The reference gets the same
// guarantee from its cooperative launch (fused/flashrnn_fused_forward.cu:893-911).  Streams under graph
// capture are left alone (a captured launch is replayed later, when this order means nothing): overlapping
// replays are the caller's to order.  Kernels of other processes are not seen; there the bounded waits and
// the status word remain the safety net.
// The event is recorded on the launching stream itself, right behind the launch (gate_leave); a later launch on
// another stream waits for that event.  `last` is only ever compared, never used: the stream it names may be gone.
struct LaunchGate { std::mutex mu; hipEvent_t ev = nullptr; hipStream_t last = nullptr; bool have = false; };
static LaunchGate g_gate[64];
static bool stream_capturing(hipStream_t st) {
  hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(st, &cs) != hipSuccess) { (void)hipGetLastError(); return false; }
  return cs != hipStreamCaptureStatusNone;
}
// Locks the device's gate and orders `st` behind the last multi-workgroup launch; returns the gate to pass to
// gate_leave, or null when there is nothing to do (one workgroup per head, capture, no device).
static LaunchGate* gate_enter(int kw, hipStream_t st) {
  if (kw <= 1) return nullptr;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
  if (stream_capturing(st)) return nullptr;
  LaunchGate* g = &g_gate[dev];
  g->mu.lock();
  if (g->have && g->last != st) {
    if (hipStreamWaitEvent(st, g->ev, 0) != hipSuccess) (void)hipGetLastError();
  }
  return g;
}
// record == false: the launch is not one that later launches should queue behind (the resident decode kernel, which
// stays on the device until its session ends)
static void gate_leave(LaunchGate* g, hipStream_t st, bool launched_ok = true, bool record = true) {
  if (!g) return;
  if (launched_ok && record) {
    if (!g->ev && hipEventCreateWithFlags(&g->ev, hipEventDisableTiming) != hipSuccess) { g->ev = nullptr; (void)hipGetLastError(); }
    if (g->ev && hipEventRecord(g->ev, st) == hipSuccess) { g->last = st; g->have = true; }
    else { g->have = false; (void)hipGetLastError(); }
  }
  g->mu.unlock();
}

// fx is the cell the kernels are instantiated for: the function itself, except that an Elman cell under
// forward_clipval runs as FRNN_ELMAN_CLIP (one cached value per element: the unclamped h).
// rc: the gate cache is left out (forward) / rebuilt (backward): only for cells that have one.
struct Opts { float h_clip, g_clip; int cut; int fx; int rc; int bs; };
static int parse_opts(const frnn_options* o, int function, Opts* out) {
  out->h_clip = 0.f; out->g_clip = 0.f; out->cut = 0; out->fx = function; out->rc = 0; out->bs = 0;
  if (!o) return 0;
  // (the struct may grow at its end: struct_size says how much of it the caller's build knows)
  if (o->struct_size < offsetof(frnn_options, recompute))
    return fail(FRNN_E_ARG, "frnn_options.struct_size = %u: set it to sizeof(frnn_options) (%zu here)", o->struct_size, sizeof(frnn_options));
  const int recompute = o->struct_size >= offsetof(frnn_options, recompute) + sizeof(int) ? o->recompute : 0;
  if (o->forward_clipval != o->forward_clipval || o->gradient_recurrent_clipval != o->gradient_recurrent_clipval ||
      o->forward_clipval < 0.f || o->gradient_recurrent_clipval < 0.f)
    return fail(FRNN_E_ARG, "clip values must be positive, or 0 for none (got %g, %g)", (double)o->forward_clipval,
                (double)o->gradient_recurrent_clipval);
  out->h_clip = o->forward_clipval; out->g_clip = o->gradient_recurrent_clipval; out->cut = o->gradient_recurrent_cut != 0;
  if (function == FRNN_ELMAN && out->h_clip > 0.f) out->fx = FRNN_ELMAN_CLIP;
  out->rc = recompute != 0 && function != FRNN_ELMAN;
  out->bs = o->struct_size >= offsetof(frnn_options, batch_stride) + sizeof(int) ? o->batch_stride : 0;
  if (out->bs < 0) return fail(FRNN_E_ARG, "batch_stride must be 0 (= B) or the number of rows of the whole batch (got %d)", out->bs);  // (elman caches nothing, or one value under forward_clipval)
  return 0;
}

struct Bump {
  unsigned char* base; size_t off;
  void* take(size_t bytes) { void* p = base ? base + off : nullptr; off += (bytes + 255) & ~(size_t)255; return p; }
};

static int check_problem(int function, int dtype, int B, int T, int N, int D) {
  if (function < 0 || function > 3) return fail(FRNN_E_ARG, "unknown function id %d", function);
  if (dtype != FRNN_BF16 && dtype != FRNN_F32 && dtype != FRNN_F16) return fail(FRNN_E_ARG, "unknown dtype id %d", dtype);
  if (B <= 0 || T <= 0 || N <= 0 || D <= 0) return fail(FRNN_E_ARG, "non-positive size B=%d T=%d N=%d D=%d", B, T, N, D);
  if ((long)B * T >= (1L << 31)) return fail(FRNN_E_ARG, "B*T too large");
  return 0;
}
// gate cache of the fused kernels: NC values per element, padded to whole dwords (CacheBlk in frnn_common.h)
static size_t fused_cache_bytes_of(int function, int dtype, int B, int T, int N, int D) {
  const int nc = cell_dims(function).NC + (cache_carried_state(function, (int)dtype_size(dtype), D) >= 0 ? 1 : 0);
  const int ncp = dtype_size(dtype) == 2 ? (nc + 1) / 2 * 2 : nc;
  return (size_t)T * N * B * D * ncp * dtype_size(dtype);
}
// the fused kernels address each tensor with 32-bit byte offsets
// bs: rows between the state planes (0: B)
static int check_fused_sizes(int function, int dtype, int B, int T, int N, int D, int bs = 0, bool with_cache = true) {
  const CellDims c = cell_dims(function);
  const size_t es = dtype_size(dtype), tnd = (size_t)T * N * D;
  if (bs != 0 && bs < B) return fail(FRNN_E_ARG, "batch_stride %d is smaller than the %d rows of the call", bs, B);
  const size_t planes = ((size_t)(c.S - 1) * (bs ? bs : B) + B) * tnd * es;  // from the first row of plane 0 to the last of plane S-1
  const size_t cache = with_cache ? fused_cache_bytes_of(function, dtype, B, T, N, D) : 0;
  if ((size_t)B * tnd * c.GW * es >= ((size_t)1 << 31) || planes >= ((size_t)1 << 31) || cache >= ((size_t)1 << 31))
    return fail(FRNN_E_TOO_LARGE, "a tensor of this call reaches 2 GiB (the fused kernels use 32-bit offsets): run the batch as ranges "
                "of at most frnn_fused_max_batch() rows (frnn_options.batch_stride lets them use the full tensors in place)");
  return 0;
}
static int check_ptr(const void* p, const char* name) {
  if (!p) return fail(FRNN_E_NULL, "%s is null", name);
  if (((uintptr_t)p) & 15) return fail(FRNN_E_ALIGN, "%s is not 16-byte aligned", name);
  return 0;
}
#define CHECK_PTR(p) { int e_ = check_ptr(p, #p); if (e_) return e_; }

// ---- fused workspace layouts --------------------------------------------------------------------
struct FusedFwdWs { int* status; u64* ll; int* xcd; size_t zero_bytes; size_t total; };
static FusedFwdWs carve_fused_fwd(void* ws, int dtype, int B, int N, int D, const Plan& p) {
  Bump bp{(unsigned char*)ws, 0};
  FusedFwdWs w;
  w.status = (int*)bp.take(256);
  const int tr = tile_rows_for(B, N, p.kw, p.waves, p.max_tr, dtype);
  const size_t groups = (size_t)N * ((B + tr - 1) / tr);
  const size_t llw = (size_t)16 * D / (dtype == FRNN_F32 ? 1 : 2);
  w.ll = (u64*)bp.take(p.kw > 1 ? groups * 3 * llw * 8 : 0);
  w.xcd = (int*)bp.take(p.kw > 1 ? groups * 32 * 4 : 0);  // words of xcd_handshake
  w.zero_bytes = bp.off;  // status, exchange slots and handshake words must start at zero for every call
#ifdef FRNN_TRACE
  bp.take(1 << 20);
#endif
  w.total = bp.off;
  return w;
}
struct FusedBwdWs { int* status; u64* ll; int* xcd; size_t zero_bytes; void* Rt; void* dgx; float* dbp; float* part; int splits; size_t total; };
static FusedBwdWs carve_fused_bwd(void* ws, int function, int dtype, int B, int T, int N, int D, const Plan& p) {
  const CellDims c = cell_dims(function);
  const size_t es = dtype_size(dtype);
  Bump bp{(unsigned char*)ws, 0};
  FusedBwdWs w;
  w.status = (int*)bp.take(256);
  const int tr = tile_rows_for(B, N, p.kw, p.waves, p.max_tr, dtype);
  const size_t bt = (B + tr - 1) / tr, groups = (size_t)N * bt;
  w.ll = (u64*)bp.take(p.kw > 1 ? groups * 3 * bwd_inbox_words(D, p.kw) * 8 : 0);
  w.xcd = (int*)bp.take(p.kw > 1 ? groups * 32 * 4 : 0);  // words of xcd_handshake
  w.zero_bytes = bp.off;
#ifdef FRNN_TRACE
  bp.take(1 << 20);
#endif
  w.Rt = bp.take((size_t)N * D * c.GR * D * es);
  w.dgx = bp.take(function == FRNN_GRU ? (size_t)B * T * N * D * es : 0);
  w.dbp = (float*)bp.take(bt * c.GT * N * D * 4);
  w.splits = grad_gemm_splits(dtype, B, T, N, D, c.GR);
  w.part = (float*)bp.take((size_t)w.splits * c.GR * N * D * D * 4);
  w.total = bp.off;
  return w;
}

template <int F> static int fused_fwd_dispatch(int dtype, const Plan& p, const FwdArgs& a, hipStream_t st) {
  return dtype == FRNN_BF16 ? fused_fwd_launch<F, FRNN_BF16>(p, a, st)
       : dtype == FRNN_F16 ? fused_fwd_launch<F, FRNN_F16>(p, a, st) : fused_fwd_launch<F, FRNN_F32>(p, a, st);
}
template <int F> static int fused_bwd_dispatch(int dtype, const Plan& p, const BwdArgs& a, hipStream_t st) {
  return dtype == FRNN_BF16 ? fused_bwd_launch<F, FRNN_BF16>(p, a, st)
       : dtype == FRNN_F16 ? fused_bwd_launch<F, FRNN_F16>(p, a, st) : fused_bwd_launch<F, FRNN_F32>(p, a, st);
}

// common tail of both backward paths: dR GEMM, final reductions
static int weight_grads(int function, int dtype, int B, int T, int N, int D, const void* s0, const void* states,
                        const void* dWx, const void* dgx, float* part, int splits, const float* dbp, int db_splits,
                        float* dR, float* db, hipStream_t st) {
  const CellDims c = cell_dims(function);
  const size_t es = dtype_size(dtype);
  const size_t ND = (size_t)N * D;
  GradGemmArgs g;
  memset(&g, 0, sizeof(g));
  for (int k = 0; k < c.GR; ++k) {
    if (function == FRNN_GRU) {
      // R gates [g, r, z]: g lives in dgx, r and z are Wx gates 0 and 1
      if (k == 0) { g.gsrc[k] = dgx; g.gld[k] = (long)ND; }
      else { g.gsrc[k] = (const char*)dWx + (size_t)(k - 1) * ND * es; g.gld[k] = (long)(c.GW * ND); }
    } else {
      g.gsrc[k] = (const char*)dWx + (size_t)k * ND * es; g.gld[k] = (long)(c.GW * ND);
    }
  }
  g.states_h = states; g.s0_h = s0; g.part = part;
  g.B = B; g.T = T; g.N = N; g.D = D; g.GR = c.GR;
  prof_begin("grad_gemm_kernel", st);
  int e = launch_grad_gemm(dtype, g, splits, st);
  prof_end(st);
  if (e) return hip_fail(e, "dR gemm");
  prof_begin("grad_reduce_kernel", st);
  e = launch_grad_reduce(part, splits, (size_t)c.GR * N * D * D, dR, dbp, db_splits, (size_t)c.GT * ND, db, st);
  prof_end(st);
  if (e) return hip_fail(e, "gradient reduction");
  return 0;
}

// ---- static scratch of frnn_fused_forward_static ------------------------------------------------------
// Workspace (status word + the exchange slots between the workgroups of a head) for callers that cannot
// allocate.  Every device the library runs on holds its own copy of the array until the process ends; in
// host code the array's name is only a handle for hipGetSymbolAddress, the address itself is looked up
// once per device (with that device current) and kept.
// The array has two areas: the first kStaticForwardBytes serve frnn_fused_forward_static, the rest is where the
// single-step kernels (frnn_fused_step) put their status word and the exchange words that nobody reads, so that a
// step on one stream cannot touch the live exchange of a static forward call on another.
static constexpr size_t kStaticScratchBytes = (size_t)4 << 20;
static constexpr size_t kStaticStepBytes = (size_t)512 << 10;
static constexpr size_t kStaticProbeBytes = 256;  // the two words of frnn_streams_overlap, at the very end
static constexpr size_t kStaticForwardBytes = kStaticScratchBytes - kStaticStepBytes - kStaticProbeBytes;
static __device__ __align__(256) unsigned char g_static_scratch[kStaticScratchBytes];
static std::mutex g_scratch_mu;
static void* g_scratch_ptr[64] = {nullptr};
static int static_scratch(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(FRNN_E_DEVICE, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= 64) return fail(FRNN_E_DEVICE, "device index %d out of range", dev);
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_static_scratch));
    if (e != hipSuccess || !p) return fail(FRNN_E_DEVICE, "hipGetSymbolAddress(static scratch): %s", hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

// ---- resident decode kernel: tiling, residency, mailbox layout ---------------------------------------------
struct DecodePlan { Plan p; MbLayout l; int groups; };
// Tiling, residency and mailbox layout of a decode session; 0 or an error code (message set).
static int decode_plan(int function, int dtype, int B, int N, int D, int slots, DecodePlan* out) {
  int e = check_problem(function, dtype, B, 1, N, D);
  if (e) return e;
  if (slots != 2 && slots != 4 && slots != 8 && slots != 16) return fail(FRNN_E_ARG, "slots must be 2, 4, 8 or 16 (got %d)", slots);
  if (!find_plan(function, dtype, D, 0, 0, &out->p))
    return fail(FRNN_E_UNSUPPORTED, "no fused kernel for function %d dtype %d head dim %d", function, dtype, D);
  const Plan& p = out->p;
  out->groups = N * ((B + 3) / 4);
  // every workgroup of the session stays on the device until the session ends: all of them must fit at once
  const long room = p.kw > 1 ? groups_per_launch(p.kw) : (long)device_cus() * (p.waves <= 4 ? 2 : 1);
  if (out->groups > room)
    return fail(FRNN_E_UNSUPPORTED, "a decode session of %d groups (N * ceil(B / 4)) does not fit the device at once (room for %ld "
                "with %d workgroup(s) per head)", out->groups, room, p.kw);
  const CellDims c = cell_dims(function);
  const size_t llw = (size_t)16 * D / (dtype == FRNN_F32 ? 1 : 2);
  out->l = mb_layout(dtype, B, N, D, c.GW, c.S, slots, p.kw > 1 ? (size_t)out->groups * 3 * llw * 8 : 0,
                     p.kw > 1 ? (size_t)out->groups * 32 * 4 : 0);
  if ((size_t)slots * out->l.in_slot >= ((size_t)1 << 31) || (size_t)slots * out->l.out_slot >= ((size_t)1 << 31))
    return fail(FRNN_E_ARG, "the inbox of this session reaches 2 GiB");
  return 0;
}
template <typename T> static int exchange_launch(int function, const MbExchangeArgs& x, dim3 grid, hipStream_t st) {
  switch (function) {
    case FRNN_LSTM:  hipLaunchKernelGGL((decode_exchange_kernel<T, 4, 2>), grid, dim3(256), 0, st, x); break;
    case FRNN_SLSTM: hipLaunchKernelGGL((decode_exchange_kernel<T, 4, 4>), grid, dim3(256), 0, st, x); break;
    case FRNN_GRU:   hipLaunchKernelGGL((decode_exchange_kernel<T, 3, 1>), grid, dim3(256), 0, st, x); break;
    default:         hipLaunchKernelGGL((decode_exchange_kernel<T, 1, 1>), grid, dim3(256), 0, st, x); break;
  }
  return (int)hipGetLastError();
}
template <int F> static int fused_dec_dispatch(int dtype, const Plan& p, const FwdArgs& a, hipStream_t st) {
  return dtype == FRNN_BF16 ? fused_dec_launch<F, FRNN_BF16>(p, a, st)
       : dtype == FRNN_F16 ? fused_dec_launch<F, FRNN_F16>(p, a, st) : fused_dec_launch<F, FRNN_F32>(p, a, st);
}
// `second` waits (on the device) for everything queued on `first` so far
static int order_streams(hipStream_t first, hipStream_t second) {
  hipEvent_t ev;
  hipError_t e = hipEventCreateWithFlags(&ev, hipEventDisableTiming);
  if (e != hipSuccess) return (int)e;
  e = hipEventRecord(ev, first);
  if (e == hipSuccess) e = hipStreamWaitEvent(second, ev, 0);
  (void)hipEventDestroy(ev);  // (the wait keeps what it needs)
  return (int)e;
}

}  // namespace frnn

using namespace frnn;

extern "C" {

const char* frnn_last_error(void) { return g_err; }
const char* frnn_version(void) { return "flashrnn_hip 0.1 (gfx950)"; }

void frnn_profile_enable(int on) { g_prof_on = on ? 1 : 0; g_prof_n = 0; }
void frnn_profile_reset(void) { g_prof_n = 0; }
int frnn_profile_count(void) { return (int)(g_prof_n < kProfMax ? g_prof_n : kProfMax); }
const char* frnn_profile_name(int i) { const int k = prof_slot(i); return k < 0 ? "" : g_prof[k].name; }
float frnn_profile_ms(int i) {
  const int k = prof_slot(i);
  if (k < 0) return -1.0f;
  float ms = -1.0f;
  if (hipEventSynchronize(g_prof[k].b) != hipSuccess) return -1.0f;
  if (hipEventElapsedTime(&ms, g_prof[k].a, g_prof[k].b) != hipSuccess) return -1.0f;
  return ms;
}

int frnn_function_dims(int function, int* G_r, int* G_w, int* G_t, int* S, int* cache_vals) {
  if (function < 0 || function > 3) return fail(FRNN_E_ARG, "unknown function id %d", function);
  const CellDims c = cell_dims(function);
  if (G_r) *G_r = c.GR;
  if (G_w) *G_w = c.GW;
  if (G_t) *G_t = c.GT;
  if (S) *S = c.S;
  if (cache_vals) *cache_vals = c.NC;
  return 0;
}

// ---- fused ----------------------------------------------------------------------------------------
int frnn_fused_supported(int function, int dtype, int B, int N, int D) {
  int e = check_problem(function, dtype, B, 1, N, D);
  if (e) return e;
  Plan pf, pb;
  if (!find_plan(function, dtype, D, 0, 0, &pf) || !find_plan(function, dtype, D, 0, 1, &pb))
    return fail(FRNN_E_UNSUPPORTED, "no fused kernel for function %d dtype %d head dim %d", function, dtype, D);
  return 0;
}

int frnn_fused_plan(int function, int dtype, int B, int N, int D, int backward,
                    int* waves, int* tiles_per_wave, int* wgs_per_head, int* active_wgs) {
  int e = check_problem(function, dtype, B, 1, N, D);
  if (e) return e;
  Plan p;
  if (!pick_plan(function, dtype, B, N, D, backward, &p))
    return fail(FRNN_E_UNSUPPORTED, "no fused kernel for function %d dtype %d head dim %d", function, dtype, D);
  if (waves) *waves = p.waves;
  if (tiles_per_wave) *tiles_per_wave = p.utw;
  if (wgs_per_head) *wgs_per_head = p.kw;
  const int tr = tile_rows_for(B, N, p.kw, p.waves, p.max_tr, dtype);
  if (active_wgs) *active_wgs = N * ((B + tr - 1) / tr) * p.kw;
  return 0;
}

size_t frnn_fused_cache_bytes(int function, int dtype, int B, int T, int N, int D) {
  if (check_problem(function, dtype, B, T, N, D)) return 0;
  return fused_cache_bytes_of(function, dtype, B, T, N, D);
}

size_t frnn_fused_cache_bytes_opt(int function, int dtype, int B, int T, int N, int D, const frnn_options* opt) {
  Opts o;
  if (check_problem(function, dtype, B, T, N, D) || parse_opts(opt, function, &o)) return 0;
  return o.rc ? 0 : fused_cache_bytes_of(o.fx, dtype, B, T, N, D);
}

int frnn_fused_max_batch(int function, int dtype, int T, int N, int D, int batch_stride, int training, const frnn_options* opt) {
  g_err[0] = 0;
  Opts o;
  if (check_problem(function, dtype, 1, T, N, D) || parse_opts(opt, function, &o) || batch_stride < 0) return 0;
  const CellDims c = cell_dims(o.fx);
  const size_t es = dtype_size(dtype), tnd = (size_t)T * N * D, lim = ((size_t)1 << 31) - 1;
  size_t rows = lim / (tnd * c.GW * es);
  const size_t cache_row = (training && !o.rc) ? fused_cache_bytes_of(o.fx, dtype, 1, T, N, D) : 0;
  if (cache_row) rows = rows < lim / cache_row ? rows : lim / cache_row;
  if (batch_stride == 0) rows = rows < lim / (tnd * es * c.S) ? rows : lim / (tnd * es * c.S);
  else {
    const size_t below = (size_t)(c.S - 1) * batch_stride * tnd * es;
    const size_t r = below >= lim ? 0 : (lim - below) / (tnd * es);
    rows = rows < r ? rows : r;
  }
  return (int)(rows > 0x3fffffff ? 0x3fffffff : rows);
}

size_t frnn_fused_workspace_bytes(int function, int dtype, int B, int T, int N, int D, int backward) {
  if (check_problem(function, dtype, B, T, N, D)) return 0;
  Plan p;
  if (!pick_plan(function, dtype, B, N, D, backward, &p)) return 0;
  return backward ? carve_fused_bwd(nullptr, function, dtype, B, T, N, D, p).total
                  : carve_fused_fwd(nullptr, dtype, B, N, D, p).total;
}

size_t frnn_fused_workspace_bytes_opt(int function, int dtype, int B, int T, int N, int D, int backward,
                                      const frnn_options* opt) {
  Opts o;
  if (check_problem(function, dtype, B, T, N, D) || parse_opts(opt, function, &o)) return 0;
  Plan p;
  if (!pick_plan(o.fx, dtype, B, N, D, backward ? (o.rc ? 2 : 1) : 0, &p)) return 0;
  return backward ? carve_fused_bwd(nullptr, o.fx, dtype, B, T, N, D, p).total
                  : carve_fused_fwd(nullptr, dtype, B, N, D, p).total;
}

int frnn_fused_forward(int function, int dtype, int training, int B, int T, int N, int D,
                       const void* Wx, const void* R, const void* b, const void* s0,
                       void* states, void* cache, void* workspace, size_t workspace_bytes, void* stream) {
  return frnn_fused_forward_opt(function, dtype, training, B, T, N, D, Wx, R, b, s0, states, cache, workspace,
                                workspace_bytes, stream, nullptr);
}

// The forward call proper.  `workspace` is the caller's buffer or this library's static scratch array.
// step != 0: one time step with carried state (frnn_fused_step): T = 1, no training, no workspace clear
// (the one step neither waits for nor reads anything in the workspace; its exchange stores land in one
// area shared by all groups), optional fp32 carry.
static int fused_forward_impl(int function, int dtype, int training, int B, int T, int N, int D,
                              const void* Wx, const void* R, const void* b, const void* s0,
                              void* states, void* cache, void* workspace, size_t workspace_bytes, void* stream,
                              const frnn_options* opt, int step = 0, float* carry = nullptr) {
  g_err[0] = 0;
  int e = check_problem(function, dtype, B, T, N, D);
  if (e) return e;
  Opts o;
  e = parse_opts(opt, function, &o);
  if (e) return e;
  const int fx = o.fx;
  Plan p;
  if (!pick_plan(fx, dtype, B, N, D, 0, &p))
    return fail(FRNN_E_UNSUPPORTED, "no fused kernel for function %d dtype %d head dim %d", function, dtype, D);
  e = check_fused_sizes(fx, dtype, B, T, N, D, o.bs, training && !o.rc);
  if (e) return e;
  CHECK_PTR(Wx) CHECK_PTR(R) CHECK_PTR(b) CHECK_PTR(s0) CHECK_PTR(states) CHECK_PTR(workspace)
  if (o.rc) {
    Plan prc;
    if (!find_plan(fx, dtype, D, 0, 2, &prc))
      return fail(FRNN_E_UNSUPPORTED, "no recompute-mode kernel for function %d dtype %d head dim %d", function, dtype, D);
  }
  const bool need_cache = training && cell_dims(fx).NC > 0 && !o.rc;
  if (need_cache) CHECK_PTR(cache)
  hipStream_t st = (hipStream_t)stream;
  FusedFwdWs w = carve_fused_fwd(workspace, dtype, B, N, D, p);
  if (!step) {
    if (workspace_bytes < w.total) return fail(FRNN_E_WORKSPACE, "workspace %zu < %zu bytes", workspace_bytes, w.total);
    if (p.kw > 1) {  // (a head of one workgroup has no exchange words, and its kernel sets the status word itself)
      prof_begin("fill_zero_kernel", st);
      e = launch_fill_zero(workspace, w.zero_bytes, st);
      prof_end(st);
      if (e) return hip_fail(e, "workspace clear");
    }
  } else {
    const size_t one_group = 256 + (p.kw > 1 ? (size_t)3 * 16 * D / (dtype == FRNN_F32 ? 1 : 2) * 8 + 256 : 0);
    if (workspace_bytes < one_group) return fail(FRNN_E_WORKSPACE, "step scratch %zu < %zu bytes", workspace_bytes, one_group);
  }
  const int tr = tile_rows_for(B, N, p.kw, p.waves, p.max_tr, dtype);
  const int groups = N * ((B + tr - 1) / tr);
  int per_launch = groups;
  if (p.kw > 1) {  // workgroups that wait for each other must all be resident
    per_launch = groups_per_launch(p.kw);
    if (per_launch < 1) return fail(FRNN_E_DEVICE, "the device has too few compute units for the %d workgroups of one head", p.kw);
  }
  FwdArgs a;
  a.Wx = Wx; a.R = R; a.b = b; a.s0 = s0; a.states = states; a.cache = cache;
  a.ll = w.ll; a.status = w.status;
  a.xcd = (near_stores_possible(p) && !step && near_stores_allowed()) ? w.xcd : nullptr;
  a.carry = carry; a.step = step;
  a.B = B; a.BS = o.bs ? o.bs : B; a.T = T; a.N = N; a.groups_total = groups; a.tile_rows = tr;
  a.training = need_cache ? 1 : 0;
  a.spin_limit = env_int("FRNN_SPIN_LIMIT", 1 << 22);
  p.cooperative = env_int("FRNN_COOPERATIVE", 0);
  a.poll_delay = env_int("FRNN_POLL_DELAY", fwd_poll_delay_default(fx, dtype, p, tr));
  a.h_clip = o.h_clip;
  a.mailbox = nullptr; a.inbox_off = a.outbox_off = a.in_slot = a.out_slot = 0; a.slots = 1; a.idle_limit = 0;
  // producer-wave stores: for launches that put some load on the memory system (measured, bf16 T = 1024, forward kernel
  // with the producer wave storing against the compute lanes storing: LSTM N12 D64 B256 0.82 against 1.03 ms, B128 0.50 / 0.65,
  // B64 0.38 / 0.38, B16 0.30 / 0.295; sLSTM N12 D64 B128 0.68 / 0.97; GRU N12 D64 B256 0.66 / 0.78; LSTM N24 D32 B256
  // 1.11 / 1.33); FRNN_PRODUCER_STORES=0/1 overrides
  a.pst = step ? 0 : env_int("FRNN_PRODUCER_STORES", tr == 4 && p.kw == 1 && 2 * groups > device_cus() ? 1 : 0);
  a.trace = nullptr;
#ifdef FRNN_TRACE
  a.trace = (long long*)((char*)workspace + w.zero_bytes);
#endif
  LaunchGate* gate = gate_enter(step ? 1 : p.kw, st);  // (the workgroups of a single step never wait for each other)
  for (int g0 = 0; g0 < groups; g0 += per_launch) {
    a.grp0 = g0; a.groups = groups - g0 < per_launch ? groups - g0 : per_launch;
    prof_begin("fused_fwd_kernel", st);
    switch (fx) {
      case FRNN_LSTM:  e = fused_fwd_dispatch<FRNN_LSTM>(dtype, p, a, st); break;
      case FRNN_SLSTM: e = fused_fwd_dispatch<FRNN_SLSTM>(dtype, p, a, st); break;
      case FRNN_GRU:   e = fused_fwd_dispatch<FRNN_GRU>(dtype, p, a, st); break;
      case FRNN_ELMAN: e = fused_fwd_dispatch<FRNN_ELMAN>(dtype, p, a, st); break;
      default:         e = fused_fwd_dispatch<FRNN_ELMAN_CLIP>(dtype, p, a, st); break;
    }
    prof_end(st);
    if (e) break;
  }
  gate_leave(gate, st, e == 0);
  return e ? hip_fail(e, "fused forward launch") : 0;
}

int frnn_fused_forward_opt(int function, int dtype, int training, int B, int T, int N, int D,
                           const void* Wx, const void* R, const void* b, const void* s0,
                           void* states, void* cache, void* workspace, size_t workspace_bytes, void* stream,
                           const frnn_options* opt) {
  return fused_forward_impl(function, dtype, training, B, T, N, D, Wx, R, b, s0, states, cache, workspace,
                            workspace_bytes, stream, opt);
}

size_t frnn_fused_forward_static_max_bytes(void) { return kStaticForwardBytes; }

int frnn_fused_forward_static(int function, int dtype, int training, int B, int T, int N, int D,
                              const void* Wx, const void* R, const void* b, const void* s0,
                              void* states, void* cache, void* stream, const frnn_options* opt) {
  g_err[0] = 0;
  // refuse what does not fit before anything else, so that the message names the limit
  int e = check_problem(function, dtype, B, T, N, D);
  if (e) return e;
  Plan p;
  if (!pick_plan(function, dtype, B, N, D, 0, &p))
    return fail(FRNN_E_UNSUPPORTED, "no fused kernel for function %d dtype %d head dim %d", function, dtype, D);
  const size_t need = carve_fused_fwd(nullptr, dtype, B, N, D, p).total;
  if (need > kStaticForwardBytes)
    return fail(FRNN_E_WORKSPACE, "this problem needs %zu bytes of workspace, the static scratch array holds %zu: "
                "use frnn_fused_forward_opt with a workspace of the caller", need, kStaticForwardBytes);
  void* ws = nullptr;
  e = static_scratch(&ws);
  if (e) return e;
  return fused_forward_impl(function, dtype, training, B, T, N, D, Wx, R, b, s0, states, cache, ws,
                            kStaticForwardBytes, stream, opt);
}

int frnn_fused_backward(int function, int dtype, int B, int T, int N, int D,
                        const void* R, const void* b, const void* s0, const void* states,
                        const void* cache, const void* dstates,
                        void* dWx, void* ds0, float* dR, float* db,
                        void* workspace, size_t workspace_bytes, void* stream) {
  return frnn_fused_backward_opt(function, dtype, B, T, N, D, R, b, s0, states, cache, dstates, dWx, ds0, dR, db,
                                 workspace, workspace_bytes, stream, nullptr);
}

// The backward call proper.  Recompute mode (opt->recompute, a cell that has a gate cache): `Wx` and `b` are
// read instead of `cache`, which is ignored.
static int fused_backward_impl(int function, int dtype, int B, int T, int N, int D,
                               const void* Wx, const void* R, const void* b, const void* s0, const void* states,
                               const void* cache, const void* dstates,
                               void* dWx, void* ds0, float* dR, float* db,
                               void* workspace, size_t workspace_bytes, void* stream, const frnn_options* opt) {
  g_err[0] = 0;
  int e = check_problem(function, dtype, B, T, N, D);
  if (e) return e;
  Opts o;
  e = parse_opts(opt, function, &o);
  if (e) return e;
  const int fx = o.fx;
  const CellDims c = cell_dims(fx);
  Plan p;
  if (!pick_plan(fx, dtype, B, N, D, o.rc ? 2 : 1, &p))
    return fail(FRNN_E_UNSUPPORTED, "no fused%s kernel for function %d dtype %d head dim %d", o.rc ? " recompute-mode" : "",
                function, dtype, D);
  e = check_fused_sizes(fx, dtype, B, T, N, D, o.bs, !o.rc);
  if (e) return e;
  CHECK_PTR(R) CHECK_PTR(s0) CHECK_PTR(states) CHECK_PTR(dstates)
  CHECK_PTR(dWx) CHECK_PTR(ds0) CHECK_PTR(dR) CHECK_PTR(db) CHECK_PTR(workspace)
  if (o.rc) { CHECK_PTR(Wx) CHECK_PTR(b) }
  else if (c.NC > 0) CHECK_PTR(cache)
  const FusedBwdWs w = carve_fused_bwd(workspace, fx, dtype, B, T, N, D, p);
  if (workspace_bytes < w.total) return fail(FRNN_E_WORKSPACE, "workspace %zu < %zu bytes", workspace_bytes, w.total);
  hipStream_t st = (hipStream_t)stream;
  if (p.kw > 1) {  // (as in the forward call)
    prof_begin("fill_zero_kernel", st);
    e = launch_fill_zero(workspace, w.zero_bytes, st);
    prof_end(st);
    if (e) return hip_fail(e, "workspace clear");
  }
  prof_begin("transpose_r_kernel", st);
  e = launch_transpose_r(dtype, R, w.Rt, N, D, c.GR, st);
  prof_end(st);
  if (e) return hip_fail(e, "R transpose");
  const int tr = tile_rows_for(B, N, p.kw, p.waves, p.max_tr, dtype);
  const int bt = (B + tr - 1) / tr, groups = N * bt;
  int per_launch = groups;
  if (p.kw > 1) {
    per_launch = groups_per_launch(p.kw);
    if (per_launch < 1) return fail(FRNN_E_DEVICE, "the device has too few compute units for the %d workgroups of one head", p.kw);
  }
  BwdArgs a;
  a.Rt = w.Rt; a.s0 = s0; a.states = states; a.cache = o.rc ? nullptr : cache; a.dstates = dstates;
  a.Wx = Wx; a.R = R; a.b = b;
  a.dWx = dWx; a.dgx = w.dgx; a.ds0 = ds0; a.dbp = w.dbp;
  a.ll = w.ll; a.status = w.status;
  a.xcd = (near_stores_possible(p) && near_stores_allowed()) ? w.xcd : nullptr;
  a.B = B; a.BS = o.bs ? o.bs : B; a.T = T; a.N = N; a.groups_total = groups; a.tile_rows = tr;
  a.spin_limit = env_int("FRNN_SPIN_LIMIT", 1 << 22);
  p.cooperative = env_int("FRNN_COOPERATIVE", 0);
  // measured best, as in the forward call (exchange stores kept in the XCD's L2): the gated cells 0-2 units at every
  // head dim from 192 to 1024 (their dWx stores are issued between the send and the first probe, which is part of
  // their delay), elman D = 512 4, D = 1024 8; recompute mode sends its first probe behind the LDS reads of the
  // rebuild: best without a delay for every cell
  a.poll_delay = env_int("FRNN_POLL_DELAY_BWD", o.rc ? 0 : c.GR == 1 ? (p.kw > 4 ? 8 : 4) : 2);
  a.g_clip = o.g_clip; a.cut = o.cut;
  // producer-wave stores of dWx, under the same condition (reverse kernel: LSTM N12 D64 B256 1.16 against 1.26 ms, B128
  // 0.64 / 0.76, B64 0.48 / 0.49, B16 0.41 / 0.41; GRU N12 D64 B256 0.79 / 0.97; sLSTM N12 D64 B128 0.80 / 1.00; LSTM N24 D32
  // B256 1.22 / 1.53.  With the stores issued in front of the loads of an iteration the same kernels lost up to 25 %:
  // a wave's memory operations complete in order, and the stores are acknowledged late)
  a.pst = env_int("FRNN_PRODUCER_STORES", tr == 4 && p.kw == 1 && 2 * groups > device_cus() ? 1 : 0);
  a.trace = nullptr;
#ifdef FRNN_TRACE
  a.trace = (long long*)((char*)workspace + w.zero_bytes);
#endif
  LaunchGate* gate = gate_enter(a.cut ? 1 : p.kw, st);  // (the truncated reverse scan exchanges nothing)
  for (int g0 = 0; g0 < groups; g0 += per_launch) {
    a.grp0 = g0; a.groups = groups - g0 < per_launch ? groups - g0 : per_launch;
    prof_begin("fused_bwd_kernel", st);
    switch (fx) {
      case FRNN_LSTM:  e = fused_bwd_dispatch<FRNN_LSTM>(dtype, p, a, st); break;
      case FRNN_SLSTM: e = fused_bwd_dispatch<FRNN_SLSTM>(dtype, p, a, st); break;
      case FRNN_GRU:   e = fused_bwd_dispatch<FRNN_GRU>(dtype, p, a, st); break;
      case FRNN_ELMAN: e = fused_bwd_dispatch<FRNN_ELMAN>(dtype, p, a, st); break;
      default:         e = fused_bwd_dispatch<FRNN_ELMAN_CLIP>(dtype, p, a, st); break;
    }
    prof_end(st);
    if (e) break;
  }
  gate_leave(gate, st, e == 0);
  if (e) return hip_fail(e, "fused backward launch");
  return weight_grads(fx, dtype, B, T, N, D, s0, states, dWx, w.dgx, w.part, w.splits, w.dbp, bt, dR, db, st);
}

int frnn_fused_backward_opt(int function, int dtype, int B, int T, int N, int D,
                            const void* R, const void* b, const void* s0, const void* states,
                            const void* cache, const void* dstates,
                            void* dWx, void* ds0, float* dR, float* db,
                            void* workspace, size_t workspace_bytes, void* stream, const frnn_options* opt) {
  if (opt && opt->struct_size >= sizeof(frnn_options) && opt->recompute && function != FRNN_ELMAN) {
    g_err[0] = 0;
    return fail(FRNN_E_ARG, "recompute mode has no gate cache: call frnn_fused_backward_recompute, which takes Wx");
  }
  return fused_backward_impl(function, dtype, B, T, N, D, nullptr, R, b, s0, states, cache, dstates, dWx, ds0, dR, db,
                             workspace, workspace_bytes, stream, opt);
}

int frnn_fused_backward_recompute(int function, int dtype, int B, int T, int N, int D,
                                  const void* Wx, const void* R, const void* b, const void* s0, const void* states,
                                  const void* dstates, void* dWx, void* ds0, float* dR, float* db,
                                  void* workspace, size_t workspace_bytes, void* stream, const frnn_options* opt) {
  frnn_options o2;
  memset(&o2, 0, sizeof(o2));
  if (opt) memcpy(&o2, opt, opt->struct_size < sizeof(o2) ? opt->struct_size : sizeof(o2));
  o2.struct_size = sizeof(o2);
  o2.recompute = 1;
  if (Wx && Wx == dWx) { g_err[0] = 0; return fail(FRNN_E_ARG, "dWx must not be Wx: the scan reads Wx two steps ahead of its dWx stores"); }
  return fused_backward_impl(function, dtype, B, T, N, D, Wx, R, b, s0, states, nullptr, dstates, dWx, ds0, dR, db,
                             workspace, workspace_bytes, stream, &o2);
}

int frnn_fused_recompute_supported(int function, int dtype, int B, int N, int D) {
  int e = frnn_fused_supported(function, dtype, B, N, D);
  if (e) return e;
  Plan p;
  if (function != FRNN_ELMAN && !find_plan(function, dtype, D, 0, 2, &p))
    return fail(FRNN_E_UNSUPPORTED, "no recompute-mode kernel for function %d dtype %d head dim %d", function, dtype, D);
  return 0;
}

// ---- resident decode kernel -------------------------------------------------------------------------------

int frnn_streams_overlap(void* stream, void* kernel_stream) {
  g_err[0] = 0;
  hipStream_t st = (hipStream_t)stream, ks = (hipStream_t)kernel_stream;
  if (st == ks) return 0;
  if (stream_capturing(st) || stream_capturing(ks)) return fail(FRNN_E_ARG, "streams under capture cannot be probed");
  void* ws = nullptr;
  int e = static_scratch(&ws);
  if (e) return e;
  int* words = (int*)(static_cast<unsigned char*>(ws) + kStaticScratchBytes - kStaticProbeBytes);
  static std::mutex mu;  // (one probe at a time: they share the two words)
  std::lock_guard<std::mutex> lk(mu);
  hipError_t h = hipStreamSynchronize(st);  // work queued on `stream` earlier must not be mistaken for the resident kernel
  if (h == hipSuccess) h = (hipError_t)launch_fill_zero(words, kStaticProbeBytes, st);
  if (h == hipSuccess) h = (hipError_t)order_streams(st, ks);
  if (h != hipSuccess) return hip_fail((int)h, "overlap probe setup");
  // a kernel that waits on `kernel_stream` (at most ~3 ms) for a word that a kernel on `stream` sets
  hipLaunchKernelGGL(overlap_spin_kernel, dim3(1), dim3(64), 0, ks, words, 20000);
  h = hipGetLastError();
  if (h == hipSuccess) { hipLaunchKernelGGL(decode_ctrl_store_kernel, dim3(1), dim3(64), 0, st, words, 1); h = hipGetLastError(); }
  int host[2] = {0, 0};
  if (h == hipSuccess) h = hipStreamSynchronize(ks);
  if (h == hipSuccess) h = hipMemcpyAsync(host, words, sizeof(host), hipMemcpyDeviceToHost, st);
  if (h == hipSuccess) h = hipStreamSynchronize(st);
  if (h != hipSuccess) return hip_fail((int)h, "overlap probe");
  return host[1] == 1 ? 1 : 0;
}

size_t frnn_fused_decode_mailbox_bytes(int function, int dtype, int B, int N, int D, int slots) {
  DecodePlan dp;
  if (decode_plan(function, dtype, B, N, D, slots, &dp)) return 0;
  return dp.l.total;
}

int frnn_fused_decode_mailbox_layout(int function, int dtype, int B, int N, int D, int slots,
                                     size_t* inbox_offset, size_t* inbox_slot_bytes,
                                     size_t* outbox_offset, size_t* outbox_slot_bytes) {
  g_err[0] = 0;
  DecodePlan dp;
  int e = decode_plan(function, dtype, B, N, D, slots, &dp);
  if (e) return e;
  if (inbox_offset) *inbox_offset = dp.l.inbox_off;
  if (inbox_slot_bytes) *inbox_slot_bytes = dp.l.in_slot;
  if (outbox_offset) *outbox_offset = dp.l.outbox_off;
  if (outbox_slot_bytes) *outbox_slot_bytes = dp.l.out_slot;
  return 0;
}

int frnn_fused_decode_open(int function, int dtype, int B, int N, int D,
                           const void* R, const void* b, const void* s_in, float* carry,
                           void* mailbox, size_t mailbox_bytes, int slots, int max_tokens, int idle_polls,
                           void* stream, void* kernel_stream, const frnn_options* opt) {
  g_err[0] = 0;
  DecodePlan dp;
  int e = decode_plan(function, dtype, B, N, D, slots, &dp);
  if (e) return e;
  Opts o;
  e = parse_opts(opt, function, &o);
  if (e) return e;
  if (max_tokens <= 0 || idle_polls <= 0) return fail(FRNN_E_ARG, "max_tokens and idle_polls must be positive (got %d, %d)", max_tokens, idle_polls);
  CHECK_PTR(R) CHECK_PTR(b) CHECK_PTR(s_in) CHECK_PTR(mailbox)
  if (((uintptr_t)mailbox) & 255) return fail(FRNN_E_ALIGN, "mailbox is not 256-byte aligned");
  if (carry && (((uintptr_t)carry) & 15)) return fail(FRNN_E_ALIGN, "carry is not 16-byte aligned");
  if (mailbox_bytes < dp.l.total) return fail(FRNN_E_WORKSPACE, "mailbox %zu < %zu bytes", mailbox_bytes, dp.l.total);
  hipStream_t st = (hipStream_t)stream, ks = (hipStream_t)kernel_stream;
  if (st == ks) return fail(FRNN_E_ARG, "kernel_stream must be a stream of its own: the resident kernel occupies it until the session ends");
  if (stream_capturing(st) || stream_capturing(ks)) return fail(FRNN_E_ARG, "a decode session cannot be opened under stream capture");
  if (env_int("FRNN_DECODE_NO_PROBE", 0) == 0) {
    e = frnn_streams_overlap(stream, kernel_stream);
    if (e < 0) return e;
    if (e == 0)
      return fail(FRNN_E_DEVICE, "kernels on `stream` do not run while one on `kernel_stream` is running (the two share a hardware "
                  "queue): pick another kernel_stream (frnn_streams_overlap tells which pairs work)");
  }
  // the mailbox starts at zero (no token has tag 0); cleared on the caller's stream, which also orders the clear in
  // front of the caller's first post, and the resident kernel behind it and behind whatever produced R, b and s_in
  e = launch_fill_zero(mailbox, dp.l.zero_bytes, st);
  if (e) return hip_fail(e, "mailbox clear");
  e = order_streams(st, ks);
  if (e) return hip_fail(e, "ordering the kernel stream behind the caller's");
  const Plan& p = dp.p;
  unsigned char* mb = static_cast<unsigned char*>(mailbox);
  FwdArgs a;
  a.Wx = nullptr; a.R = R; a.b = b; a.s0 = s_in; a.states = nullptr; a.cache = nullptr;
  a.ll = (u64*)(mb + dp.l.exch_off); a.status = (int*)mb + MB_STATUS;
  a.xcd = (near_stores_possible(p) && near_stores_allowed()) ? (int*)(mb + dp.l.xcd_off) : nullptr;
  a.carry = carry; a.step = 0;
  a.B = B; a.BS = B; a.T = max_tokens; a.N = N; a.grp0 = 0; a.groups = dp.groups; a.groups_total = dp.groups; a.tile_rows = 4;
  a.training = 0;
  a.spin_limit = env_int("FRNN_SPIN_LIMIT", 1 << 22);
  a.poll_delay = env_int("FRNN_POLL_DELAY", fwd_poll_delay_default(function, dtype, p, 4));
  a.h_clip = o.h_clip; a.pst = 0;
  a.mailbox = mailbox; a.inbox_off = dp.l.inbox_off; a.outbox_off = dp.l.outbox_off;
  a.in_slot = dp.l.in_slot; a.out_slot = dp.l.out_slot; a.slots = slots; a.idle_limit = idle_polls;
  a.trace = nullptr;
  LaunchGate* gate = gate_enter(p.kw, ks);
  switch (function) {
    case FRNN_LSTM:  e = fused_dec_dispatch<FRNN_LSTM>(dtype, p, a, ks); break;
    case FRNN_SLSTM: e = fused_dec_dispatch<FRNN_SLSTM>(dtype, p, a, ks); break;
    case FRNN_GRU:   e = fused_dec_dispatch<FRNN_GRU>(dtype, p, a, ks); break;
    default:         e = fused_dec_dispatch<FRNN_ELMAN>(dtype, p, a, ks); break;
  }
  gate_leave(gate, ks, e == 0, false);
  return e ? hip_fail(e, "resident decode kernel launch") : 0;
}

int frnn_fused_decode_step(int function, int dtype, int B, int N, int D, int count,
                           const void* Wx, void* s_out, void* mailbox, size_t mailbox_bytes, int slots, void* stream) {
  g_err[0] = 0;
  DecodePlan dp;
  int e = decode_plan(function, dtype, B, N, D, slots, &dp);
  if (e) return e;
  if (count <= 0 || count > slots) return fail(FRNN_E_ARG, "count must be between 1 and slots = %d (got %d)", slots, count);
  CHECK_PTR(Wx) CHECK_PTR(s_out) CHECK_PTR(mailbox)
  if (mailbox_bytes < dp.l.total) return fail(FRNN_E_WORKSPACE, "mailbox %zu < %zu bytes", mailbox_bytes, dp.l.total);
  MbExchangeArgs x;
  x.Wx = Wx; x.s_out = s_out; x.mailbox = mailbox;
  x.inbox_off = dp.l.inbox_off; x.outbox_off = dp.l.outbox_off; x.in_slot = dp.l.in_slot; x.out_slot = dp.l.out_slot;
  x.B = B; x.N = N; x.D = D; x.count = count; x.slots = slots;
  x.spin_limit = env_int("FRNN_SPIN_LIMIT", 1 << 22);
  const dim3 grid((unsigned)(((size_t)B * N * D + 255) / 256));
  hipStream_t st = (hipStream_t)stream;
  prof_begin("decode_exchange_kernel", st);
  e = dtype == FRNN_BF16 ? exchange_launch<bf16_t>(function, x, grid, st)
    : dtype == FRNN_F16 ? exchange_launch<half_t>(function, x, grid, st) : exchange_launch<float>(function, x, grid, st);
  prof_end(st);
  return e ? hip_fail(e, "decode exchange launch") : 0;
}

int frnn_fused_decode_close(void* mailbox, void* stream, void* kernel_stream) {
  g_err[0] = 0;
  CHECK_PTR(mailbox)
  hipStream_t st = (hipStream_t)stream, ks = (hipStream_t)kernel_stream;
  if (st == ks) return fail(FRNN_E_ARG, "kernel_stream must differ from stream");
  hipLaunchKernelGGL(decode_ctrl_store_kernel, dim3(1), dim3(64), 0, st, (int*)mailbox + MB_STOP, 1);
  int e = (int)hipGetLastError();
  if (e) return hip_fail(e, "stop word");
  e = order_streams(ks, st);  // what follows on the caller's stream sees the carry and the control block
  return e ? hip_fail(e, "ordering the caller's stream behind the resident kernel") : 0;
}

// ---- alternating --------------------------------------------------------------------------------------
int frnn_alt_supported(int function, int dtype, int B, int N, int D) {
  int e = check_problem(function, dtype, B, 1, N, D);
  if (e) return e;
  if (D % 32 != 0) return fail(FRNN_E_UNSUPPORTED, "alternating kernels need a head dim that is a multiple of 32 (got %d)", D);
  return 0;
}

size_t frnn_alt_cache_bytes(int function, int dtype, int B, int T, int N, int D) {
  if (check_problem(function, dtype, B, T, N, D)) return 0;
  return (size_t)T * B * N * D * cell_dims(function).NC * dtype_size(dtype);
}

size_t frnn_alt_cache_bytes_opt(int function, int dtype, int B, int T, int N, int D, const frnn_options* opt) {
  Opts o;
  if (check_problem(function, dtype, B, T, N, D) || parse_opts(opt, function, &o)) return 0;
  return (size_t)T * B * N * D * cell_dims(o.fx).NC * dtype_size(dtype);
}

namespace {
struct AltWs { float* sfp; void* Rt; void* dgx; void* dg; float* dsr; float* dbp; int bsplits; float* part; int splits; size_t total; };
AltWs carve_alt(void* ws, int function, int dtype, int B, int T, int N, int D, int backward) {
  const CellDims c = cell_dims(function);
  const size_t es = dtype_size(dtype), ND = (size_t)N * D, BND = (size_t)B * ND;
  Bump bp{(unsigned char*)ws, 0};
  AltWs w;
  memset(&w, 0, sizeof(w));
  if (!backward) {
    w.sfp = (float*)bp.take(BND * c.S * 4);
  } else {
    w.Rt = bp.take(ND * c.GR * D * es);
    w.dgx = bp.take(function == FRNN_GRU ? (size_t)T * BND * es : 0);
    w.dg = bp.take(2 * BND * c.GR * es);
    w.dsr = (float*)bp.take((size_t)c.S * BND * 4);
    const long rows = (long)B * T;
    w.bsplits = rows < 256 ? (int)rows : 256;
    w.dbp = (float*)bp.take((size_t)w.bsplits * c.GT * ND * 4);
    w.splits = grad_gemm_splits(dtype, B, T, N, D, c.GR);
    w.part = (float*)bp.take((size_t)w.splits * c.GR * ND * D * 4);
  }
  w.total = bp.off;
  return w;
}
}  // namespace

size_t frnn_alt_workspace_bytes(int function, int dtype, int B, int T, int N, int D, int backward) {
  if (check_problem(function, dtype, B, T, N, D)) return 0;
  return carve_alt(nullptr, function, dtype, B, T, N, D, backward).total;
}

int frnn_alt_forward(int function, int dtype, int training, int B, int T, int N, int D,
                     const void* Wx, const void* R, const void* b, const void* s0,
                     void* states, void* cache, void* workspace, size_t workspace_bytes, void* stream) {
  return frnn_alt_forward_opt(function, dtype, training, B, T, N, D, Wx, R, b, s0, states, cache, workspace,
                              workspace_bytes, stream, nullptr);
}

int frnn_alt_forward_opt(int function, int dtype, int training, int B, int T, int N, int D,
                         const void* Wx, const void* R, const void* b, const void* s0,
                         void* states, void* cache, void* workspace, size_t workspace_bytes, void* stream,
                         const frnn_options* opt) {
  g_err[0] = 0;
  int e = frnn_alt_supported(function, dtype, B, N, D);
  if (e) return e;
  Opts o;
  e = parse_opts(opt, function, &o);
  if (e) return e;
  if (T <= 0) return fail(FRNN_E_ARG, "non-positive T=%d", T);
  CHECK_PTR(Wx) CHECK_PTR(R) CHECK_PTR(b) CHECK_PTR(s0) CHECK_PTR(states) CHECK_PTR(workspace)
  const bool need_cache = training && cell_dims(o.fx).NC > 0;
  if (need_cache) CHECK_PTR(cache)
  const AltWs w = carve_alt(workspace, o.fx, dtype, B, T, N, D, 0);
  if (workspace_bytes < w.total) return fail(FRNN_E_WORKSPACE, "workspace %zu < %zu bytes", workspace_bytes, w.total);
  AltProblem p{o.fx, dtype, B, T, N, D, need_cache ? 1 : 0, o.h_clip, 0.f, 0, 0};
  AltFwdBuffers bf{Wx, R, b, s0, states, cache, w.sfp};
  prof_begin("alt_forward_steps", (hipStream_t)stream);
  e = alt_forward(p, bf, (hipStream_t)stream);
  prof_end((hipStream_t)stream);
  return e ? hip_fail(e, "alternating forward launch") : 0;
}

// ---- single step with carried state -----------------------------------------------------------------
int frnn_fused_step(int function, int dtype, int B, int N, int D,
                    const void* Wx_t, const void* R, const void* b, const void* s_in, void* s_out,
                    float* carry, void* stream, const frnn_options* opt) {
  g_err[0] = 0;
  if (s_in == s_out && s_in) return fail(FRNN_E_ARG, "s_out must not be s_in: every workgroup of a head reads all of h");
  if (carry && (((uintptr_t)carry) & 15)) return fail(FRNN_E_ALIGN, "carry is not 16-byte aligned");
  void* ws = nullptr;
  int e = static_scratch(&ws);
  if (e) return e;
  return fused_forward_impl(function, dtype, 0, B, 1, N, D, Wx_t, R, b, s_in, s_out, nullptr,
                            static_cast<unsigned char*>(ws) + kStaticForwardBytes, kStaticStepBytes, stream, opt, 1, carry);
}

int frnn_alt_step(int function, int dtype, int B, int N, int D,
                  const void* Wx_t, const void* R, const void* b, const void* s_in, void* s_out,
                  float* carry, void* stream, const frnn_options* opt) {
  g_err[0] = 0;
  int e = frnn_alt_supported(function, dtype, B, N, D);
  if (e) return e;
  Opts o;
  e = parse_opts(opt, function, &o);
  if (e) return e;
  CHECK_PTR(Wx_t) CHECK_PTR(R) CHECK_PTR(b) CHECK_PTR(s_in) CHECK_PTR(s_out)
  if (s_in == s_out) return fail(FRNN_E_ARG, "s_out must not be s_in: every workgroup of a head reads all of h");
  if (carry && (((uintptr_t)carry) & 15)) return fail(FRNN_E_ALIGN, "carry is not 16-byte aligned");
  AltProblem p{o.fx, dtype, B, 1, N, D, 0, o.h_clip, 0.f, 0, carry ? 1 : 0};
  AltFwdBuffers bf{Wx_t, R, b, s_in, s_out, nullptr, carry};
  prof_begin("alt_forward_steps", (hipStream_t)stream);
  e = alt_forward(p, bf, (hipStream_t)stream);
  prof_end((hipStream_t)stream);
  return e ? hip_fail(e, "alternating step launch") : 0;
}

int frnn_alt_backward(int function, int dtype, int B, int T, int N, int D,
                      const void* R, const void* b, const void* s0, const void* states,
                      const void* cache, const void* dstates,
                      void* dWx, void* ds0, float* dR, float* db,
                      void* workspace, size_t workspace_bytes, void* stream) {
  return frnn_alt_backward_opt(function, dtype, B, T, N, D, R, b, s0, states, cache, dstates, dWx, ds0, dR, db,
                               workspace, workspace_bytes, stream, nullptr);
}

int frnn_alt_backward_opt(int function, int dtype, int B, int T, int N, int D,
                          const void* R, const void* b, const void* s0, const void* states,
                          const void* cache, const void* dstates,
                          void* dWx, void* ds0, float* dR, float* db,
                          void* workspace, size_t workspace_bytes, void* stream, const frnn_options* opt) {
  g_err[0] = 0;
  (void)b;
  int e = frnn_alt_supported(function, dtype, B, N, D);
  if (e) return e;
  Opts o;
  e = parse_opts(opt, function, &o);
  if (e) return e;
  if (T <= 0) return fail(FRNN_E_ARG, "non-positive T=%d", T);
  const int fx = o.fx;
  const CellDims c = cell_dims(fx);
  CHECK_PTR(R) CHECK_PTR(s0) CHECK_PTR(states) CHECK_PTR(dstates)
  CHECK_PTR(dWx) CHECK_PTR(ds0) CHECK_PTR(dR) CHECK_PTR(db) CHECK_PTR(workspace)
  if (c.NC > 0) CHECK_PTR(cache)
  const AltWs w = carve_alt(workspace, fx, dtype, B, T, N, D, 1);
  if (workspace_bytes < w.total) return fail(FRNN_E_WORKSPACE, "workspace %zu < %zu bytes", workspace_bytes, w.total);
  hipStream_t st = (hipStream_t)stream;
  e = launch_transpose_r(dtype, R, w.Rt, N, D, c.GR, st);
  if (e) return hip_fail(e, "R transpose");
  AltProblem p{fx, dtype, B, T, N, D, 1, 0.f, o.g_clip, o.cut, 0};
  AltBwdBuffers bf{w.Rt, s0, states, cache, dstates, dWx, w.dgx, ds0, w.dg, w.dsr};
  prof_begin("alt_backward_steps", st);
  e = alt_backward_scan(p, bf, st);
  prof_end(st);
  if (e) return hip_fail(e, "alternating backward launch");
  // bias partial sums over (b,t) rows; sources per bias gate
  const size_t es = dtype_size(dtype), ND = (size_t)N * D;
  const void* src[4];
  long ld[4];
  for (int g = 0; g < c.GT; ++g) {
    if (fx == FRNN_GRU) {
      if (g == 0) { src[g] = w.dgx; ld[g] = (long)ND; }
      else { src[g] = (const char*)dWx + (size_t)(g - 1) * ND * es; ld[g] = (long)(c.GW * ND); }
    } else {
      src[g] = (const char*)dWx + (size_t)g * ND * es; ld[g] = (long)(c.GW * ND);
    }
  }
  prof_begin("alt_bias_kernel", st);
  e = launch_bias_partial(dtype, src, ld, c.GT, N, D, (long)B * T, w.bsplits, w.dbp, st);
  prof_end(st);
  if (e) return hip_fail(e, "bias partial sums");
  return weight_grads(fx, dtype, B, T, N, D, s0, states, dWx, w.dgx, w.part, w.splits, w.dbp, w.bsplits, dR, db, st);
}

}  // extern "C"
