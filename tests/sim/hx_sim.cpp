// Run time of the host execution model declared in hx_sim.h: fibers, the wave / workgroup scheduler, the cross-lane
// instructions, the DMA queues, guarded operand buffers.  Test infrastructure only.
#include "hx_sim.h"

#include <cxxabi.h>
#include <dlfcn.h>
#include <signal.h>
#include <stdarg.h>
#include <stdlib.h>
#include <sys/mman.h>
#include <unistd.h>

#include <string>
#include <vector>

extern "C" void hx_sim_switch(void** save_sp, void* new_sp);
// saves the callee-saved registers of the running context on its stack, stores its stack pointer, adopts the other one
asm(R"(
.text
.globl hx_sim_switch
.type hx_sim_switch,@function
hx_sim_switch:
  pushq %rbp
  pushq %rbx
  pushq %r12
  pushq %r13
  pushq %r14
  pushq %r15
  movq %rsp, (%rdi)
  movq %rsi, %rsp
  popq %r15
  popq %r14
  popq %r13
  popq %r12
  popq %rbx
  popq %rbp
  ret
.size hx_sim_switch,.-hx_sim_switch
)");

extern "C" char __start_hx_lds[], __stop_hx_lds[];

namespace hxsim {

enum { RUNNABLE, COLL, BARRIER, DONE };
enum { C_SYNC, C_DMA, C_WAIT, C_RFL, C_BALLOT, C_SHFL, C_DPP, C_SWAP, C_MFMA, C_TR };

struct Dma {
  const uint8_t* src;
  uint8_t* dst;
  int bytes;
  bool idem;  // re-fetch of what the destination already holds (see C_DMA)
};

struct Lane {
  void* sp;
  int state, tid, ckind, csite;
  Idx3 tid3;
  const void *a, *b, *c;  // operands of the pending cross-lane instruction (they live in the lane's own frame)
  void* d;
  int i0, i1;
  uint32_t u0, u1;
  Dma t;  // this lane's share of the DMA instruction it is issuing
  int stores;  // global stores this lane has executed since its wave's last cross-lane instruction
};

struct Wave {
  // the wave's vmcnt-counted instructions in issue order: a DMA instruction (the vector holds its lanes' transfers) or a
  // global store (an empty vector: it only occupies a place in the count - on this chip stores and loads share the
  // counter and retire in order, so a store issued after a DMA makes a later counted wait reach less far back)
  std::vector<std::vector<Dma>> q;
  size_t landed;  // instructions [0, landed) have completed
};

struct Config {
  int dma_lazy = 0;    // 0: a DMA lands when it is issued; 1: when the wave's vmcnt wait (or its end) forces it
  int wave_order = 0;  // 0: waves 0, 1, 2 ..; 1: the other way round
  int interleave = 0;  // 0: a wave runs until it blocks at a barrier; 1: the waves take turns after every cross-lane instruction
  int wg_reverse = 0;  // 1: the workgroups of a launch run last to first (workgroup 0 is NOT the first to start)
  int poison_lds = 1;  // fill the LDS with 0xFF (NaN in e4m3, bf16, f16 and f32) before every workgroup
};

Lane* cur = nullptr;
Geometry geo;
static Config cfg;
static void* sched_sp;
static const std::function<void()>* body;
static std::vector<Lane> lanes;
static std::vector<Wave> waves;
static uint8_t* stacks;
static const size_t STACK = 512 << 10;
static const int MAX_LANES = 1024;
static bool faulted;
static bool sched_ctx;  // `cur` names a lane only for attribution: the code runs on the scheduler's own stack
static std::string fault_msg;
static const void* launch_fn;
static std::string kernel_name() {
  Dl_info info;
  if (launch_fn && dladdr(launch_fn, &info) && info.dli_sname) {
    int st = 0;
    char* d = abi::__cxa_demangle(info.dli_sname, nullptr, nullptr, &st);
    std::string s = st == 0 && d ? d : info.dli_sname;
    free(d);
    const size_t paren = s.find('(');
    return paren == std::string::npos ? s : s.substr(0, paren);
  }
  return "?";
}
static uint64_t n_coll, n_dma, n_barrier, ticks;
// work counters of the launches since the last hx_sim_work_reset: wave-level MFMA instructions, bytes moved by DMA, LDS
// bytes read / written by ordinary and transposing accesses, workgroup barriers, workgroups
static uint64_t w_mfma, w_dma_bytes, w_lds_read, w_lds_write, w_barriers, w_workgroups;
// DMA bytes of the running workgroup that are issued and not yet covered by a wait of the issuing wave (what the code
// lets be in flight); over the launches since the last reset: the largest value, and its sum / count right after every wait
static uint64_t fly_bytes, w_fly_max, w_fly_after_wait, w_waits;
static const uint8_t *fly_lo, *fly_hi;  // if set: only transfers whose source lies in [fly_lo, fly_hi) are counted

struct Buf {
  uint8_t* base;  // first usable byte
  size_t bytes;
  uint8_t* map;
  size_t map_bytes;
};
static std::vector<Buf> bufs;

const Idx3& thread_idx() { return cur->tid3; }

static void yield_to_scheduler() { hx_sim_switch(&cur->sp, sched_sp); }

static void fail(const char* fmt, ...) {
  if (!faulted) {
    char msg[600];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(msg, sizeof msg, fmt, ap);
    va_end(ap);
    char where[200] = "";
    if (cur)
      snprintf(where, sizeof where, " [kernel %s, workgroup (%u,%u,%u), work-item %d]", kernel_name().c_str(), geo.block_idx.x,
               geo.block_idx.y, geo.block_idx.z, cur->tid);
    fault_msg = std::string(msg) + where;
    faulted = true;
  }
  if (cur && !sched_ctx) {
    void* dummy;
    hx_sim_switch(&dummy, sched_sp);  // this work-item never runs again
  }
}

static std::string describe_address(const void* p, size_t n = 1) {
  const uint8_t* a = (const uint8_t*)p;
  for (const Buf& b : bufs)
    if (a >= b.base && a < b.base + b.bytes && a + n > b.base + b.bytes) a = b.base + b.bytes;  // starts inside, runs over the end
  char s[300];
  for (size_t i = 0; i < bufs.size(); ++i) {
    const Buf& b = bufs[i];
    if (a >= b.map && a < b.map + b.map_bytes) {
      if (a < b.base) snprintf(s, sizeof s, "%ld bytes before the start of operand buffer %zu (%zu bytes)", (long)(b.base - a), i, b.bytes);
      else if (a >= b.base + b.bytes) snprintf(s, sizeof s, "%ld bytes past the end of operand buffer %zu (%zu bytes)", (long)(a - (b.base + b.bytes)), i, b.bytes);
      else snprintf(s, sizeof s, "inside operand buffer %zu", i);
      return s;
    }
  }
  snprintf(s, sizeof s, "not near any operand buffer");
  return s;
}

static bool in_a_buffer(const void* p, size_t n) {
  const uint8_t* a = (const uint8_t*)p;
  for (const Buf& b : bufs)
    if (a >= b.base && a + n <= b.base + b.bytes) return true;
  return false;
}

static void on_segv(int sig, siginfo_t* si, void*) {
  if (!cur) {  // not inside a work-item: a defect of the model itself or of the test
    signal(sig, SIG_DFL);
    raise(sig);
    return;
  }
  fail("global memory access out of bounds: address %p is %s", si->si_addr, describe_address(si->si_addr).c_str());
}

static void lane_entry() {
  (*body)();
  Lane* l = cur;
  l->state = DONE;
  yield_to_scheduler();
  abort();  // a finished work-item is never resumed
}

static void init_lane(Lane& l, int tid, dim3 block) {
  l.tid = tid;
  l.tid3 = {tid % block.x, (tid / block.x) % block.y, tid / (block.x * block.y)};
  l.state = RUNNABLE;
  l.stores = 0;
  uint64_t* top = (uint64_t*)(stacks + (size_t)(tid + 1) * STACK);
  // layout read by hx_sim_switch: six registers, then the address it returns to; the entry function then sees the
  // stack alignment of an ordinary call
  top[-1] = 0;
  top[-2] = (uint64_t)(void*)&lane_entry;
  for (int i = 3; i <= 8; ++i) top[-i] = 0;
  l.sp = (void*)(top - 8);
}

static void collective(int kind, int site) {
  cur->ckind = kind;
  cur->csite = site;
  cur->state = COLL;
  yield_to_scheduler();
}

// ---- LDS access discipline -----------------------------------------------------------------------------------------
// The kernel objects are compiled with load / store tracing (the compiler calls __sanitizer_cov_load*/store* with the
// address of every memory access), so the model sees every LDS access, not only the DMA and the transposing reads it
// executes itself, and can check the one rule the hardware gives: two accesses to the same LDS bytes from different
// waves, at least one of them a write, are ordered only by a workgroup barrier between them; and a DMA transfer writes
// its bytes at some unknown moment between its issue and the wave's vmcnt wait that covers it.  Per 4-byte word of the
// LDS the model keeps the last writer (wave, barrier epoch), the readers of the current epoch and whether a DMA into it is
// in flight; an access that is not ordered against those by a barrier (or, within one wave, by program order) is
// reported with the kernel, the workgroup, both waves and the LDS offset.  Lanes of one wave execute together and are
// never checked against each other.
struct Shadow {
  uint32_t wepoch, repoch;  // epoch of the last write / of the reads in rmask; 0 = never
  uint16_t rmask;           // waves that read it in epoch repoch
  uint8_t wwave;            // wave of the last write
  uint8_t inflight;         // 1 + wave of the DMA in flight into it, 0 = none
};
static Shadow* shadow;           // one entry per 4 bytes of the LDS section
static uint32_t epoch = 1;       // barrier epoch of the running workgroup
static bool check_lds = true;
static size_t dirty_lo = ~(size_t)0, dirty_hi = 0;  // LDS bytes written by the running workgroup (what to poison again)
static uint64_t n_lds_checked;

static void lds_race(const char* what, size_t off, int w, const Shadow& s) {
  fail("LDS race: %s at LDS offset %zu by wave %d in barrier epoch %u (last write: wave %d epoch %u; readers of epoch %u: mask 0x%x; DMA in "
       "flight from wave %d)",
       what, off, w, epoch, (int)s.wwave, s.wepoch, s.repoch, (unsigned)s.rmask, (int)s.inflight - 1);
}
enum { ACC_READ, ACC_WRITE, ACC_DMA_ISSUE, ACC_DMA_LAND };
static void lds_access(const void* p, size_t n, int kind) {
  const size_t off = (const char*)p - __start_hx_lds;
  if (kind != ACC_READ) {
    if (off < dirty_lo) dirty_lo = off;
    if (off + n > dirty_hi) dirty_hi = off + n;
  }
  if (kind == ACC_READ) w_lds_read += n;
  else if (kind == ACC_WRITE) w_lds_write += n;
  else if (kind == ACC_DMA_ISSUE) w_dma_bytes += n;
  if (!check_lds || !cur) return;
  const int w = cur->tid >> 6;
  ++n_lds_checked;
  for (size_t i = off >> 2; i <= (off + n - 1) >> 2; ++i) {
    Shadow& s = shadow[i];
    const bool other_writer = s.wepoch == epoch && s.wwave != w;
    const bool other_reader = s.repoch == epoch && (s.rmask & ~(1u << w)) != 0;
    switch (kind) {
      case ACC_READ:
        if (s.inflight) return lds_race(s.inflight - 1 == w ? "read of bytes whose DMA has not been waited for" : "read of bytes another wave's DMA is still writing", i * 4, w, s);
        if (other_writer) return lds_race("read of bytes another wave wrote since the last barrier", i * 4, w, s);
        if (s.repoch != epoch) s.repoch = epoch, s.rmask = 0;
        s.rmask |= (uint16_t)(1u << w);
        break;
      case ACC_WRITE:
        if (s.inflight) return lds_race("write to bytes a DMA is still writing", i * 4, w, s);
        if (other_writer) return lds_race("write to bytes another wave wrote since the last barrier", i * 4, w, s);
        if (other_reader) return lds_race("write to bytes another wave read since the last barrier", i * 4, w, s);
        s.wepoch = epoch, s.wwave = (uint8_t)w;
        break;
      case ACC_DMA_ISSUE:
        if (s.inflight) return lds_race("DMA into bytes another DMA is still writing", i * 4, w, s);
        if (other_writer) return lds_race("DMA into bytes another wave wrote since the last barrier", i * 4, w, s);
        if (other_reader) return lds_race("DMA into bytes another wave read since the last barrier", i * 4, w, s);
        s.inflight = (uint8_t)(w + 1);
        break;
      case ACC_DMA_LAND:
        s.inflight = 0;
        if (other_reader) return lds_race("DMA waited for in the epoch in which another wave already read its bytes", i * 4, w, s);
        s.wepoch = epoch, s.wwave = (uint8_t)w;
        break;
    }
  }
}
static bool in_a_buffer(const void* p, size_t n);
static inline void traced(const void* p, size_t n, bool write) {
  if ((const char*)p >= __start_hx_lds && (const char*)p < __stop_hx_lds) lds_access(p, n, write ? ACC_WRITE : ACC_READ);
  else if (write && cur && !sched_ctx && in_a_buffer(p, n)) ++cur->stores;  // a store to an operand: one vmcnt-counted instruction
}

// ---- DMA ----------------------------------------------------------------------------------------------------------
static Lane* checker_lane;  // a lane of the wave on whose behalf the scheduler touches the LDS (DMA issue / landing)
static void land_until(Wave& w, size_t upto) {
  for (; w.landed < upto; ++w.landed)
    for (const Dma& t : w.q[w.landed]) {
      memcpy(t.dst, t.src, t.bytes);
      if (!fly_lo || (t.src >= fly_lo && t.src < fly_hi)) fly_bytes -= t.bytes;
      if (checker_lane && !t.idem) {
        Lane* keep = cur;
        cur = checker_lane, sched_ctx = true;
        lds_access(t.dst, t.bytes, ACC_DMA_LAND);
        cur = keep, sched_ctx = false;
      }
    }
}

uint32_t lds_addr(const void* p) {
  const char* c = (const char*)p;
  if (c < __start_hx_lds || c > __stop_hx_lds) fail("hx_lds_addr: %p is not in the LDS", p);
  return (uint32_t)(c - __start_hx_lds);
}
static uint8_t* lds_ptr(uint32_t addr, int bytes, const char* what) {
  if ((size_t)addr + bytes > (size_t)(__stop_hx_lds - __start_hx_lds)) fail("%s: LDS address %u (+%d) is outside the LDS", what, addr, bytes);
  return (uint8_t*)__start_hx_lds + addr;
}

void dma(const void* gptr, uint32_t lds_dst, int bytes) {
  ++n_dma;
  if (!bufs.empty() && !in_a_buffer(gptr, bytes))
    fail("global->LDS DMA reads %d bytes at %p out of bounds: %s", bytes, gptr, describe_address(gptr, bytes).c_str());
  cur->t = Dma{(const uint8_t*)gptr, lds_ptr(lds_dst, bytes, "global->LDS DMA"), bytes, false};
  collective(C_DMA, 0);  // one wave instruction: the active lanes' transfers travel (and are waited for) together
}

// s_waitcnt: the wave goes on once at most vmcnt of its DMA instructions are still in flight (the model counts DMA
// only; the loads and stores the compiler issues share the hardware's counter, which can only make a wait stronger)
void waitcnt(int imm) {
  cur->i0 = (imm & 15) | (((imm >> 14) & 3) << 4);
  collective(C_WAIT, 0);
}

void sleep(int) { ++ticks; }
uint64_t clock100mhz() { return ++ticks; }

// ---- blocking points ---------------------------------------------------------------------------------------------
void barrier() {
  cur->i0 = 0;
  cur->state = BARRIER;
  yield_to_scheduler();
}
int barrier_or(int pred) {  // __syncthreads_or
  cur->i0 = pred != 0;
  cur->state = BARRIER;
  yield_to_scheduler();
  return cur->i1;
}


void wave_sync(int site) { collective(C_SYNC, site); }
int readfirstlane(int v, int site) {
  cur->i0 = v;
  collective(C_RFL, site);
  return cur->i1;
}
uint64_t ballot(bool p, int site) {
  cur->i0 = p;
  uint64_t r = 0;
  cur->d = &r;
  collective(C_BALLOT, site);
  return r;
}
uint32_t shfl_xor_u32(uint32_t v, int mask, int site) {
  cur->u0 = v;
  cur->i0 = mask;
  collective(C_SHFL, site);
  return cur->u1;
}
uint32_t mov_dpp_u32(uint32_t v, int ctrl, int row_mask, int bank_mask, bool bound_ctrl, int site) {
  if (ctrl < 0 || ctrl > 0xFF || row_mask != 0xF || bank_mask != 0xF) fail("DPP control 0x%x (row mask 0x%x, bank mask 0x%x) is not modelled: quad_perm only", ctrl, row_mask, bank_mask);
  (void)bound_ctrl;
  cur->u0 = v;
  cur->i0 = ctrl;
  collective(C_DPP, site);
  return cur->u1;
}
void permlane32_swap_u32(uint32_t a, uint32_t b, uint32_t out[2], int site) {
  cur->u0 = a;
  cur->u1 = b;
  cur->d = out;
  collective(C_SWAP, site);
}
void mfma(int kind, const void* a, const void* b, const void* c, void* d, int site) {
  cur->a = a;
  cur->b = b;
  cur->c = c;
  cur->d = d;
  cur->i0 = kind;
  collective(C_MFMA, site);
}
void ds_read_tr(int elem_bytes, const void* p, void* out8, int site) {
  const char* c = (const char*)p;
  if (c < __start_hx_lds || c + 8 > __stop_hx_lds) fail("transposing LDS read: %p is outside the LDS", p);
  if ((uintptr_t)p & 7) fail("transposing LDS read: address %p is not 8-byte aligned", p);
  lds_access(p, 8, ACC_READ);
  cur->a = p;
  cur->d = out8;
  cur->i0 = elem_bytes;
  collective(C_TR, site);
}

// ---- number formats --------------------------------------------------------------------------------------------------
static float e4m3_table[256];
static void init_tables() {
  for (int code = 0; code < 256; ++code) {
    const int s = code >> 7, e = (code >> 3) & 15, m = code & 7;
    float v;
    if (e == 15 && m == 7) v = NAN;
    else if (e == 0) v = ldexpf((float)m / 8.f, -6);
    else v = ldexpf(1.f + (float)m / 8.f, e - 7);
    e4m3_table[code] = s ? -v : v;
  }
}
float cvt_f32_fp8(int v, int sel) { return e4m3_table[(v >> (8 * sel)) & 0xFF]; }

// v_cvt_pk_fp8_f32 in OCP mode: round to nearest even; what rounds beyond 448 becomes NaN (e4m3fn has no infinity),
// as does NaN; values that round to below the smallest subnormal's half become (signed) zero
static uint8_t f32_to_e4m3(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  const uint8_t sign = (u >> 24) & 0x80;
  const float a = fabsf(f);
  if (!(a == a)) return sign | 0x7F;
  if (a > 464.f) return sign | 0x7F;  // 464 is the midpoint between 448 and the (absent) next value; it rounds to even = 448
  if (a == 464.f) return sign | 0x7E;
  // a <= 464: scale so that the target grid is the integers, round to nearest even there
  int e;
  frexpf(a, &e);                 // a = m * 2^e, m in [0.5, 1)
  int exp = e - 1;               // a in [2^exp, 2^(exp+1))
  if (exp < -6) exp = -6;        // subnormal range shares the exponent of the smallest normal
  const float step = ldexpf(1.f, exp - 3);
  const float q = nearbyintf(a / step);  // default rounding mode: to nearest even
  const float r = q * step;
  if (r == 0.f) return sign;
  int e2;
  const float m2 = frexpf(r, &e2);  // r = m2 * 2^e2
  int be = e2 - 1 + 7;              // biased exponent if normal
  if (be <= 0) {                    // subnormal: r = mant/8 * 2^-6
    const int mant = (int)(r / ldexpf(1.f, -9));
    return sign | (uint8_t)mant;
  }
  const int mant = (int)((m2 * 2.f - 1.f) * 8.f);
  const int code = (be << 3) | mant;
  return sign | (uint8_t)(code > 0x7E ? 0x7E : code);
}
int cvt_pk_fp8(float a, float b, int old, bool hi) {
  const uint32_t pair = (uint32_t)f32_to_e4m3(a) | ((uint32_t)f32_to_e4m3(b) << 8);
  const uint32_t o = (uint32_t)old;
  return (int)(hi ? ((o & 0x0000FFFFu) | (pair << 16)) : ((o & 0xFFFF0000u) | pair));
}
static float bf16_to_f32(uint16_t h) {
  const uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static float f16_to_f32(uint16_t h) {
  const int s = h >> 15, e = (h >> 10) & 31, m = h & 1023;
  float v;
  if (e == 31) v = m ? NAN : INFINITY;
  else if (e == 0) v = ldexpf((float)m, -24);
  else v = ldexpf(1.f + (float)m / 1024.f, e - 15);
  return s ? -v : v;
}

// D[i][j] = sum_k A[i][k] * Bt[k][j] in double (every product of two e4m3 or two 16-bit values is exact there, and so is
// the sum of an fp8 MFMA's 64 or 128 of them): rows of D stay in registers, the inner loop runs along j
__attribute__((target_clones("avx2", "default"))) static void mfma_product(int MN, int K, const double (*A)[128], const double (*Bt)[32],
                                                                           double (*D)[32]) {
  for (int i = 0; i < MN; ++i) {
    double acc[32] = {0};
    for (int k = 0; k < K; ++k) {
      const double a = A[i][k];
      for (int j = 0; j < 32; ++j) acc[j] += a * Bt[k][j];
    }
    for (int j = 0; j < MN; ++j) D[i][j] = acc[j];
  }
}

// ---- evaluation of one cross-lane instruction for the lanes `g` (indices into `lanes`) of one wave --------------------
static void resolve(int wave_first, const std::vector<int>& g) {
  Lane& first = lanes[g[0]];
  ++n_coll;
  {  // the global stores the wave executed since its last cross-lane instruction take their places in the vmcnt order
    Wave& w = waves[wave_first / 64];
    int k = 0;
    for (int i = wave_first; i < wave_first + 64 && i < (int)lanes.size(); ++i) k = std::max(k, lanes[i].stores), lanes[i].stores = 0;
    for (int i = 0; i < k; ++i) w.q.emplace_back();
  }
  auto lane_of = [&](int pos) -> Lane* {  // the group's lane at position `pos` of the wave, or null if it is not in the group
    for (int id : g)
      if (id - wave_first == pos) return &lanes[id];
    return nullptr;
  };
  switch (first.ckind) {
    case C_SYNC:
      break;
    case C_DMA: {
      // (issue and landing are checked the same way whether the data is copied now or at the wait: the in-flight mark
      // stays until the wave's wait covers the instruction)
      Wave& w = waves[wave_first / 64];
      w.q.emplace_back();  // (the new instruction is w.q.back(); the ones before it and not yet landed are in flight)
      for (int id : g) {
        Dma& t = lanes[id].t;
        // A transfer of exactly what its destination already holds, with no other transfer into those bytes in flight,
        // changes nothing whenever it lands (the kernels that keep issuing DMA past their last tile re-fetch that tile
        // into its own slot): it counts as an instruction for the waits and is otherwise left out of the access check.
        bool quiet = memcmp(t.dst, t.src, t.bytes) == 0;
        for (size_t i = (size_t)((char*)t.dst - __start_hx_lds) >> 2; quiet && i <= (size_t)((char*)t.dst - __start_hx_lds + t.bytes - 1) >> 2; ++i)
          quiet = shadow[i].inflight == 0;
        // ... and so does a second copy of a transfer of this wave that is still in flight (same source, same destination)
        for (size_t qi = w.landed; !quiet && qi + 1 < w.q.size(); ++qi)
          for (const Dma& o : w.q[qi])
            if (o.src == t.src && o.dst == t.dst && o.bytes == t.bytes) quiet = true;
        t.idem = quiet;
        w.q.back().push_back(t);
        if (!fly_lo || (t.src >= fly_lo && t.src < fly_hi)) fly_bytes += t.bytes;
        if (fly_bytes > w_fly_max) w_fly_max = fly_bytes;
        if (quiet) w_dma_bytes += t.bytes;
        if (!quiet) {
          cur = &lanes[id], sched_ctx = true;
          lds_access(t.dst, t.bytes, ACC_DMA_ISSUE);
          cur = nullptr, sched_ctx = false;
        }
        if (!cfg.dma_lazy) memcpy(t.dst, t.src, t.bytes);
      }
      break;
    }
    case C_WAIT: {
      Wave& w = waves[wave_first / 64];
      for (int id : g)
        if (lanes[id].i0 != first.i0) {
          fail("s_waitcnt: the lanes of a wave disagree on the count");
          return;
        }
      const size_t keep = (size_t)first.i0;
      checker_lane = &first;
      if (w.q.size() > keep) land_until(w, w.q.size() - keep);
      checker_lane = nullptr;
      w_fly_after_wait += fly_bytes, ++w_waits;
      break;
    }
    case C_RFL:
      for (int id : g) lanes[id].i1 = first.i0;
      break;
    case C_BALLOT: {
      uint64_t m = 0;
      for (int id : g)
        if (lanes[id].i0) m |= 1ull << (id - wave_first);
      for (int id : g) *(uint64_t*)lanes[id].d = m;
      break;
    }
    case C_SHFL:
      for (int id : g) {
        Lane* src = lane_of((id - wave_first) ^ lanes[id].i0);
        lanes[id].u1 = src ? src->u0 : lanes[id].u0;
      }
      break;
    case C_DPP:
      for (int id : g) {
        const int pos = id - wave_first, ctrl = lanes[id].i0;
        Lane* src = lane_of((pos & ~3) | ((ctrl >> (2 * (pos & 3))) & 3));
        lanes[id].u1 = src ? src->u0 : 0;
      }
      break;
    case C_SWAP: {
      // v_permlane32_swap vdst, vsrc: lanes 32..63 of vdst and lanes 0..31 of vsrc change places
      if (g.size() != 64) {
        fail("v_permlane32_swap with %zu of 64 lanes active is not modelled", g.size());
        return;
      }
      uint32_t a[64], b[64];
      for (int p = 0; p < 64; ++p) a[p] = lanes[wave_first + p].u0, b[p] = lanes[wave_first + p].u1;
      for (int p = 0; p < 64; ++p) {
        uint32_t* o = (uint32_t*)lanes[wave_first + p].d;
        o[0] = p < 32 ? a[p] : b[p - 32];
        o[1] = p < 32 ? a[p + 32] : b[p];
      }
      break;
    }
    case C_TR: {
      if (g.size() != 64) {
        fail("transposing LDS read with %zu of 64 lanes active is not modelled", g.size());
        return;
      }
      const int eb = first.i0, per = 8 / eb;  // elements each lane supplies and receives
      for (int grp = 0; grp < 4; ++grp) {
        uint8_t in[16][8];
        for (int i = 0; i < 16; ++i) memcpy(in[i], lanes[wave_first + 16 * grp + i].a, 8);
        for (int i = 0; i < 16; ++i) {
          uint8_t out[8];
          // the 16 lanes supply a [per rows][16 columns] block, each lane `per` consecutive elements of one row; lane i
          // receives column i
          for (int e = 0; e < per; ++e) memcpy(out + e * eb, &in[e * (16 / per) + i / per][(i % per) * eb], eb);
          memcpy(lanes[wave_first + 16 * grp + i].d, out, 8);
        }
      }
      break;
    }
    case C_MFMA: {
      if (g.size() != 64) {
        fail("MFMA with %zu of 64 lanes active", g.size());
        return;
      }
      ++w_mfma;
      const int kind = first.i0;
      const bool f8 = kind == MFMA_F8_32x32x64 || kind == MFMA_F8_16x16x128 || kind == MFMA_F8_16x16x32;
      const bool big = kind == MFMA_F8_32x32x64 || kind == MFMA_BF16_32x32x16 || kind == MFMA_F16_32x32x16;
      const bool bf = kind == MFMA_BF16_32x32x16 || kind == MFMA_BF16_16x16x32;
      const int MN = big ? 32 : 16;              // rows of A = columns of B
      const int KL = f8 && kind != MFMA_F8_16x16x32 ? 32 : 8;  // k values one lane supplies
      const int K = KL * (64 / MN);
      static double A[32][128], Bt[128][32], D[32][32];  // A[i][k], B transposed to [k][j], D = A B
      for (int p = 0; p < 64; ++p) {
        const Lane& l = lanes[wave_first + p];
        const int r = p % MN, k0 = (p / MN) * KL;
        for (int k = 0; k < KL; ++k) {
          if (f8) {
            A[r][k0 + k] = e4m3_table[((const uint8_t*)l.a)[k]];
            Bt[k0 + k][r] = e4m3_table[((const uint8_t*)l.b)[k]];
          } else {
            const uint16_t ha = ((const uint16_t*)l.a)[k], hb = ((const uint16_t*)l.b)[k];
            A[r][k0 + k] = bf ? bf16_to_f32(ha) : f16_to_f32(ha);
            Bt[k0 + k][r] = bf ? bf16_to_f32(hb) : f16_to_f32(hb);
          }
        }
      }
      mfma_product(MN, K, A, Bt, D);
      const int NR = big ? 16 : 4;  // results per lane
      for (int p = 0; p < 64; ++p) {
        Lane& l = lanes[wave_first + p];
        const int j = p % MN;  // column of D (from operand B)
        float out[16];
        for (int r = 0; r < NR; ++r) {
          const int i = big ? 8 * (r / 4) + 4 * (p / 32) + (r % 4) : 4 * (p / 16) + r;  // row of D (from operand A)
          out[r] = (float)((double)((const float*)l.c)[r] + D[i][j]);
        }
        memcpy(l.d, out, NR * 4);
      }
      break;
    }
    default:
      fail("unknown cross-lane instruction %d", first.ckind);
      return;
  }
  for (int id : g) lanes[id].state = RUNNABLE;
}

static void run_lane(Lane& l) {
  cur = &l;
  hx_sim_switch(&sched_sp, l.sp);
  cur = nullptr;
}

// runs the wave until all its lanes wait at a barrier or are finished (or, with cfg.interleave, until it has completed
// one cross-lane instruction); returns whether anything ran
static bool run_wave(int first, int count) {
  bool progress = false;
  std::vector<int> g;
  while (!faulted) {
    for (int i = first; i < first + count && !faulted; ++i)
      if (lanes[i].state == RUNNABLE) {
        run_lane(lanes[i]);
        progress = true;
      }
    if (faulted) break;
    int lead = -1;
    for (int i = first; i < first + count; ++i)
      if (lanes[i].state == COLL) {
        lead = i;
        break;
      }
    if (lead < 0) break;
    g.clear();
    for (int i = first; i < first + count; ++i)
      if (lanes[i].state == COLL && lanes[i].ckind == lanes[lead].ckind && lanes[i].csite == lanes[lead].csite) g.push_back(i);
    resolve(first, g);
    progress = true;
    if (cfg.interleave) break;
  }
  return progress;
}

static void run_workgroup(dim3 block) {
  const int n = (int)(block.x * block.y * block.z);
  // what the previous workgroup wrote is poisoned again (0xFF: NaN in every format the kernels use), so a read of LDS
  // bytes this workgroup has not written shows up in the results; and every workgroup starts its own barrier epochs
  if (dirty_hi > dirty_lo) {
    if (cfg.poison_lds) memset(__start_hx_lds + dirty_lo, 0xFF, dirty_hi - dirty_lo);
    memset(shadow + (dirty_lo >> 2), 0, (((dirty_hi - 1) >> 2) - (dirty_lo >> 2) + 1) * sizeof(Shadow));  // incl. in-flight marks of a stopped launch
  }
  dirty_lo = ~(size_t)0, dirty_hi = 0;
  epoch += 2;
  ++w_workgroups;
  fly_bytes = 0;
  lanes.resize(n);
  for (int i = 0; i < n; ++i) init_lane(lanes[i], i, block);
  const int nwaves = (n + 63) / 64;
  waves.assign(nwaves, Wave{{}, 0});
  while (!faulted) {
    bool progress = false;
    for (int k = 0; k < nwaves && !faulted; ++k) {
      const int w = cfg.wave_order ? nwaves - 1 - k : k;
      progress |= run_wave(w * 64, std::min(64, n - w * 64));
    }
    if (faulted) break;
    int done = 0, at_barrier = 0;
    for (const Lane& l : lanes) done += l.state == DONE, at_barrier += l.state == BARRIER;
    if (done == n) break;
    if (done + at_barrier == n) {  // every wave that still runs has arrived
      ++n_barrier;
      ++w_barriers;
      ++epoch;
      int any = 0;
      for (const Lane& l : lanes)
        if (l.state == BARRIER) any |= l.i0;
      for (Lane& l : lanes)
        if (l.state == BARRIER) l.state = RUNNABLE, l.i1 = any;
      continue;
    }
    if (!progress) {
      fail("deadlock: %d work-items finished, %d at a barrier, %d waiting elsewhere", done, at_barrier, n - done - at_barrier);
      break;
    }
  }
  if (!faulted)
    for (size_t wi = 0; wi < waves.size(); ++wi) land_until(waves[wi], waves[wi].q.size());  // transfers in flight at the end do complete
}

hipError_t run(dim3 grid, dim3 block, const std::function<void()>& fn, const void* kernel) {
  static bool once = false;
  if (!once) {
    once = true;
    init_tables();
    stacks = (uint8_t*)mmap(nullptr, (size_t)MAX_LANES * STACK, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
    if (stacks == (uint8_t*)MAP_FAILED) abort();
    const size_t lds_bytes = __stop_hx_lds - __start_hx_lds;
    shadow = (Shadow*)mmap(nullptr, (lds_bytes / 4 + 1) * sizeof(Shadow), PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
    if (shadow == (Shadow*)MAP_FAILED) abort();
    memset(__start_hx_lds, 0xFF, lds_bytes);
    struct sigaction sa;
    memset(&sa, 0, sizeof sa);
    sa.sa_sigaction = on_segv;
    sa.sa_flags = SA_SIGINFO | SA_NODEFER;
    sigaction(SIGSEGV, &sa, nullptr);
    sigaction(SIGBUS, &sa, nullptr);
    if (const char* e = getenv("HX_SIM_DMA_LAZY")) cfg.dma_lazy = atoi(e);
    if (const char* e = getenv("HX_SIM_WAVE_ORDER")) cfg.wave_order = atoi(e);
    if (const char* e = getenv("HX_SIM_INTERLEAVE")) cfg.interleave = atoi(e);
    if (const char* e = getenv("HX_SIM_CHECK_LDS")) check_lds = atoi(e) != 0;
  }
  const long nthreads = (long)block.x * block.y * block.z;
  if (nthreads < 1 || nthreads > MAX_LANES || grid.x < 1 || grid.y < 1 || grid.z < 1) {
    launch_fn = kernel;
    fault_msg = std::string("invalid launch geometry for ") + kernel_name();
    return hipErrorLaunchFailure;
  }
  if (faulted) return hipErrorLaunchFailure;  // a fault is sticky until hx_sim_reset, like a device fault is
  body = &fn;
  launch_fn = kernel;
  static const bool trace = getenv("HX_SIM_TRACE_LAUNCHES") != nullptr;  // one line per launch on stderr
  if (trace) fprintf(stderr, "[hx_sim] launch %s grid (%u,%u,%u) block %ld\n", kernel_name().c_str(), grid.x, grid.y, grid.z, nthreads);
  geo.block_dim = {block.x, block.y, block.z};
  geo.grid_dim = {grid.x, grid.y, grid.z};
  const unsigned long total = (unsigned long)grid.x * grid.y * grid.z;
  for (unsigned long i = 0; i < total && !faulted; ++i) {
    const unsigned long id = cfg.wg_reverse ? total - 1 - i : i;
    geo.block_idx = {(unsigned)(id % grid.x), (unsigned)((id / grid.x) % grid.y), (unsigned)(id / ((unsigned long)grid.x * grid.y))};
    run_workgroup(block);
  }
  body = nullptr;
  return faulted ? hipErrorLaunchFailure : hipSuccess;
}

}  // namespace hxsim

const char* hipGetErrorString(hipError_t e) { return e == hipSuccess ? "no error" : hxsim::fault_msg.c_str(); }
// The modelled chip has 256 CUs unless a test asks for fewer (1 .. 63), which makes the code paths that depend on the
// ratio of work items to CUs (several column groups per workgroup, tickets, k splits) reachable at small sizes.  The
// library caches the CU count per device id, so every setting is its own device id.
static int sim_cus = 256;
hipError_t hipGetDevice(int* dev) {
  *dev = sim_cus % 64;
  return hipSuccess;
}
hipError_t hipDeviceGetAttribute(int* value, hipDeviceAttribute_t, int) {
  *value = sim_cus;
  return hipSuccess;
}

// ---- the compiler's load / store tracing calls (kernel objects only are built with tracing) ------------------------------
extern "C" {
void __sanitizer_cov_load1(uint8_t* p) { hxsim::traced(p, 1, false); }
void __sanitizer_cov_load2(uint16_t* p) { hxsim::traced(p, 2, false); }
void __sanitizer_cov_load4(uint32_t* p) { hxsim::traced(p, 4, false); }
void __sanitizer_cov_load8(uint64_t* p) { hxsim::traced(p, 8, false); }
void __sanitizer_cov_load16(__int128* p) { hxsim::traced(p, 16, false); }
void __sanitizer_cov_store1(uint8_t* p) { hxsim::traced(p, 1, true); }
void __sanitizer_cov_store2(uint16_t* p) { hxsim::traced(p, 2, true); }
void __sanitizer_cov_store4(uint32_t* p) { hxsim::traced(p, 4, true); }
void __sanitizer_cov_store8(uint64_t* p) { hxsim::traced(p, 8, true); }
void __sanitizer_cov_store16(__int128* p) { hxsim::traced(p, 16, true); }
void __sanitizer_cov_8bit_counters_init(char*, char*) {}
void __sanitizer_cov_pcs_init(const uintptr_t*, const uintptr_t*) {}
}

// ---- C interface for the tests ---------------------------------------------------------------------------------------
extern "C" {
void hx_sim_work(uint64_t out[9], int reset) {
  out[0] = hxsim::w_mfma, out[1] = hxsim::w_dma_bytes, out[2] = hxsim::w_lds_read, out[3] = hxsim::w_lds_write;
  out[4] = hxsim::w_barriers, out[5] = hxsim::w_workgroups;
  out[6] = hxsim::w_fly_max, out[7] = hxsim::w_fly_after_wait, out[8] = hxsim::w_waits;
  if (reset) {
    hxsim::w_mfma = hxsim::w_dma_bytes = hxsim::w_lds_read = hxsim::w_lds_write = hxsim::w_barriers = hxsim::w_workgroups = 0;
    hxsim::w_fly_max = hxsim::w_fly_after_wait = hxsim::w_waits = 0;
  }
}
void hx_sim_in_flight_source(const void* p, size_t bytes) {  // (nullptr: every transfer counts)
  hxsim::fly_lo = (const uint8_t*)p, hxsim::fly_hi = (const uint8_t*)p + bytes;
}
int hx_sim_set_check_lds(int on) {
  const int old = hxsim::check_lds;
  hxsim::check_lds = on != 0;
  return old;
}
// An operand buffer of `bytes` usable bytes between two inaccessible pages.  end_flush != 0: the last byte sits right
// before the trailing page (an overrun of one byte faults); otherwise the first byte sits right after the leading page.
void* hx_sim_alloc(size_t bytes, int end_flush) {
  // 1 MiB of inaccessible address space either side, so that an access a few rows off still lands in it
  const size_t page = 4096, guard = 256 * page, body = (bytes + page - 1) / page * page, total = body + 2 * guard;
  uint8_t* m = (uint8_t*)mmap(nullptr, total, PROT_NONE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
  if (m == (uint8_t*)MAP_FAILED) return nullptr;
  if (body) mprotect(m + guard, body, PROT_READ | PROT_WRITE);
  uint8_t* base = end_flush ? m + guard + body - bytes : m + guard;
  if (end_flush) base = (uint8_t*)((uintptr_t)base & ~(uintptr_t)15);  // keep the 16-byte alignment the kernels ask of operands
  hxsim::bufs.push_back({base, bytes, m, total});
  return base;
}
void hx_sim_free_all() {
  for (auto& b : hxsim::bufs) munmap(b.map, b.map_bytes);
  hxsim::bufs.clear();
}
// dma_lazy, wave_order, interleave: see hxsim::Config; a negative value leaves the setting as it is
void hx_sim_config(int dma_lazy, int wave_order, int interleave) {
  if (dma_lazy >= 0) hxsim::cfg.dma_lazy = dma_lazy;
  if (wave_order >= 0) hxsim::cfg.wave_order = wave_order;
  if (interleave >= 0) hxsim::cfg.interleave = interleave;
}
int hx_sim_set_wg_reverse(int on) {
  const int old = hxsim::cfg.wg_reverse;
  hxsim::cfg.wg_reverse = on != 0;
  return old;
}
int hx_sim_set_cus(int n) {
  const int old = sim_cus;
  if (n == 256 || (n >= 1 && n <= 63)) sim_cus = n;
  return old;
}
const char* hx_sim_last_fault() { return hxsim::fault_msg.c_str(); }
void hx_sim_reset() {
  hxsim::faulted = false;
  hxsim::fault_msg.clear();
}
void hx_sim_counters(uint64_t out[4]) {
  out[0] = hxsim::n_coll;
  out[1] = hxsim::n_dma;
  out[2] = hxsim::n_barrier;
  out[3] = hxsim::n_lds_checked;
}
// the conversions, for direct tests against the oracle's codec
int hx_sim_cvt_pk_fp8(float a, float b) {
  hxsim::init_tables();
  return hxsim::cvt_pk_fp8(a, b, 0, false) & 0xFFFF;
}
}
