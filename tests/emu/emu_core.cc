// TEST INFRASTRUCTURE: CPU emulator behind tests/emu/shim/hip/hip_runtime.h.  One fiber per GPU lane, blocks of a
// launch one after the other.  Fibers run until they reach a rendezvous (a wave-wide operation or a barrier); a
// wave-wide operation is carried out when every lane of the wave that is still running has arrived at it.  Lanes of
// a wave are therefore NOT in lockstep between rendezvous points: code that exchanges data between lanes through LDS
// without a barrier needs __builtin_amdgcn_wave_barrier() (a rendezvous here, no instruction on the GPU).
// Divergence: when every running fiber of a block is waiting and a wave's lanes wait at different call sites, the
// group at the lowest code address goes first (the taken side of a structured `if` precedes the join point).
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <sys/mman.h>

#include <vector>

#include "../../include/bgmoe.h"

extern "C" void emu_switch(void** save_sp, void* load_sp);
asm(R"(
.text
.globl emu_switch
.type emu_switch,@function
emu_switch:
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
.size emu_switch, .-emu_switch
)");

void emu_install_handlers();

namespace emu {
namespace {

enum Op { OP_NONE = 0, OP_SYNC, OP_SHFL, OP_BALLOT, OP_RFL, OP_RLANE, OP_MFMA16_F8, OP_MFMA32_F8, OP_MFMA16_BF16, OP_DPP, OP_BARRIER };

struct Pending { const uint8_t* src; uint8_t* dst; unsigned bytes; };

struct Fiber {
  Lane lane;
  void* sp = nullptr;
  uint8_t* stack = nullptr;
  bool done = false;
  Op op = OP_NONE;                 // what the fiber waits at (OP_NONE: runnable)
  const void* site = nullptr;
  uint32_t in[40];
  uint32_t out[16];
  std::vector<Pending> pending;    // lazy asynchronous loads, oldest first
  uint32_t async_seq = 0;
};

constexpr size_t kStack = 256 * 1024;
constexpr int kMaxThreads = 1024;

std::vector<Fiber> g_fibers;
std::vector<uint8_t*> g_stacks;
Fiber* g_cur = nullptr;
void* g_sched_sp = nullptr;
const std::function<void()>* g_body = nullptr;
alignas(256) uint8_t g_dynamic_lds[160 * 1024];
extern "C" uint8_t __start_emu_lds[], __stop_emu_lds[];     // the kernels' static __shared__ objects (linker symbols)
__attribute__((section("emu_lds"), used)) uint8_t g_lds_section_anchor[16];   // the section exists whatever is staged
bool g_lazy = false;
int g_wait_slack = 0;          // tests of the model itself: every wait_vm<N>(), N > 0, lets this many more loads stay out
bool g_count_plain = false;     // lazy model: ordinary global loads take a place in the queue too
size_t g_dynamic_bytes = 0;         // dynamic LDS the running launch asked for
int g_schedule = 0;
uint64_t g_stat_launches = 0, g_stat_blocks = 0, g_stat_rendezvous = 0, g_stat_async = 0;
struct UniformTag { uint32_t seq; const void* base; uint32_t lds; bool used; };
std::vector<UniformTag> g_uniform;   // [wave][slot]: what the first lane of a wave passed for its seq-th async load
constexpr int kUniformSlots = 64;

[[noreturn]] void die(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  fprintf(stderr, "emu: ");
  vfprintf(stderr, fmt, ap);
  fprintf(stderr, "\n");
  va_end(ap);
  fflush(stderr);
  abort();
}

void fiber_main() {
  (*g_body)();
  Fiber* f = g_cur;
  for (const Pending& p : f->pending)
    if (p.bytes) memcpy(p.dst, p.src, p.bytes);                          // whatever was still in flight lands
  f->pending.clear();
  f->done = true;
  emu_switch(&f->sp, g_sched_sp);
  die("a finished fiber was resumed");
}

void yield_to_scheduler() {
  Fiber* f = g_cur;
  emu_switch(&f->sp, g_sched_sp);
}

float bf16_to_f32(uint16_t b) {
  const uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

// carries out the operation the fibers [first, first + n) of one wave wait at (all at the same site), for the
// lanes in `who`
void perform(Fiber* wave, const std::vector<int>& who) {
  const Op op = wave[who[0]].op;
  ++g_stat_rendezvous;
  switch (op) {
    case OP_SYNC:
    case OP_BARRIER:
      break;
    case OP_SHFL:
    case OP_RLANE:
      for (int l : who) {
        const int src = (int)(wave[l].in[1] & 63u);
        bool present = false;
        for (int m : who) present = present || m == src;
        wave[l].out[0] = present ? wave[src].in[0] : wave[l].in[0];
      }
      break;
    case OP_BALLOT: {
      uint64_t m = 0;
      for (int l : who) m |= (uint64_t)(wave[l].in[0] != 0) << l;
      for (int l : who) { wave[l].out[0] = (uint32_t)m; wave[l].out[1] = (uint32_t)(m >> 32); }
      break;
    }
    case OP_RFL:
      for (int l : who) wave[l].out[0] = wave[who[0]].in[0];
      break;
    case OP_DPP:
      // in: old, src, ctrl, row mask, bank mask, bound_ctrl.  A lane whose row (16 lanes) or bank (4 lanes) is masked
      // out, or whose source lane does not exist or is not taking part, keeps `old` (0 with bound_ctrl).
      for (int l : who) {
        const int ctrl = (int)wave[l].in[2], rows = (int)wave[l].in[3], banks = (int)wave[l].in[4];
        const int row = l >> 4, in_row = l & 15;
        int src = -1;
        if (ctrl < 0x100) src = (l & ~3) | ((ctrl >> (2 * (l & 3))) & 3);          // quad_perm
        else if (ctrl == 0x140) src = (row << 4) | (15 - in_row);                    // row_mirror
        else if (ctrl == 0x141) src = (row << 4) | (in_row & 8) | (7 - (in_row & 7));  // row_half_mirror
        else if (ctrl == 0x142) src = row >= 1 ? ((row - 1) << 4) | 15 : -1;         // row_bcast15
        else if (ctrl == 0x143) src = row >= 2 ? 31 : -1;                            // row_bcast31
        else die("DPP control 0x%x is not emulated", ctrl);
        bool present = false;
        for (int m : who) present = present || m == src;
        const bool enabled = ((rows >> row) & 1) && ((banks >> (in_row >> 2)) & 1);
        if (enabled && present) wave[l].out[0] = wave[src].in[1];
        else wave[l].out[0] = (enabled && wave[l].in[5]) ? 0u : wave[l].in[0];
      }
      break;
    case OP_MFMA16_F8: {
      // A: lane l = row l % 16, K bytes 32 (l / 16) .. + 31; B likewise with its column; D[i][j]: lane j + 16 (i / 4),
      // register i % 4
      if (who.size() != 64) die("matrix instruction with %zu of 64 lanes", who.size());
      float A[16][128], B[16][128];
      for (int l = 0; l < 64; ++l) {
        const uint8_t* a = reinterpret_cast<const uint8_t*>(wave[l].in);
        const uint8_t* b = reinterpret_cast<const uint8_t*>(wave[l].in + 8);
        for (int k = 0; k < 32; ++k) {
          A[l & 15][32 * (l >> 4) + k] = e4m3_to_f32(a[k]);
          B[l & 15][32 * (l >> 4) + k] = e4m3_to_f32(b[k]);
        }
      }
      for (int l = 0; l < 64; ++l)
        for (int r = 0; r < 4; ++r) {
          const int i = 4 * (l >> 4) + r, j = l & 15;
          float c;
          memcpy(&c, &wave[l].in[16 + r], 4);
          float s = 0.0f;
          for (int k = 0; k < 128; ++k) s += A[i][k] * B[j][k];
          const float d = c + s;
          memcpy(&wave[l].out[r], &d, 4);
        }
      break;
    }
    case OP_MFMA32_F8: {
      // A: lane l = row l % 32, K bytes 32 (l / 32) .. + 31; B likewise; D[i][j]: lane j + 32 ((i / 4) % 2),
      // register 4 (i / 8) + i % 4
      if (who.size() != 64) die("matrix instruction with %zu of 64 lanes", who.size());
      static float A[32][64], B[32][64];
      for (int l = 0; l < 64; ++l) {
        const uint8_t* a = reinterpret_cast<const uint8_t*>(wave[l].in);
        const uint8_t* b = reinterpret_cast<const uint8_t*>(wave[l].in + 8);
        for (int k = 0; k < 32; ++k) {
          A[l & 31][32 * (l >> 5) + k] = e4m3_to_f32(a[k]);
          B[l & 31][32 * (l >> 5) + k] = e4m3_to_f32(b[k]);
        }
      }
      for (int l = 0; l < 64; ++l)
        for (int v = 0; v < 16; ++v) {
          const int i = 8 * (v >> 2) + 4 * (l >> 5) + (v & 3), j = l & 31;
          float c;
          memcpy(&c, &wave[l].in[16 + v], 4);
          float s = 0.0f;
          for (int k = 0; k < 64; ++k) s += A[i][k] * B[j][k];
          const float d = c + s;
          memcpy(&wave[l].out[v], &d, 4);
        }
      break;
    }
    case OP_MFMA16_BF16: {
      // A: lane l = row l % 16, K elements 8 (l / 16) .. + 7; B likewise; D as the 16x16 form above
      if (who.size() != 64) die("matrix instruction with %zu of 64 lanes", who.size());
      float A[16][32], B[16][32];
      for (int l = 0; l < 64; ++l) {
        const uint16_t* a = reinterpret_cast<const uint16_t*>(wave[l].in);
        const uint16_t* b = reinterpret_cast<const uint16_t*>(wave[l].in + 4);
        for (int k = 0; k < 8; ++k) {
          A[l & 15][8 * (l >> 4) + k] = bf16_to_f32(a[k]);
          B[l & 15][8 * (l >> 4) + k] = bf16_to_f32(b[k]);
        }
      }
      for (int l = 0; l < 64; ++l)
        for (int r = 0; r < 4; ++r) {
          const int i = 4 * (l >> 4) + r, j = l & 15;
          float c;
          memcpy(&c, &wave[l].in[8 + r], 4);
          float s = 0.0f;
          for (int k = 0; k < 32; ++k) s += A[i][k] * B[j][k];
          const float d = c + s;
          memcpy(&wave[l].out[r], &d, 4);
        }
      break;
    }
    default:
      die("unknown rendezvous %d", (int)op);
  }
  for (int l : who) wave[l].op = OP_NONE;
}

// the lanes of `wave` (nl of them) that still run all wait at one wave-wide operation at one site: carry it out
bool try_wave(Fiber* wave, int nl) {
  const void* site = nullptr;
  Op op = OP_NONE;
  std::vector<int> who;
  for (int l = 0; l < nl; ++l) {
    if (wave[l].done) continue;
    if (wave[l].op == OP_NONE || wave[l].op == OP_BARRIER) return false;
    if (who.empty()) { site = wave[l].site; op = wave[l].op; }
    else if (wave[l].site != site || wave[l].op != op) return false;
    who.push_back(l);
  }
  if (who.empty()) return false;
  perform(wave, who);
  return true;
}

// rendezvous of the calling lane: deposit is done, wait until the operation has been carried out
void rendezvous(Op op, const void* site) {
  Fiber* f = g_cur;
  f->op = op;
  f->site = site;
  if (op != OP_BARRIER) {
    Fiber* wave = &g_fibers[f->lane.wave * 64];
    const int nl = (int)std::min<size_t>(64, g_fibers.size() - f->lane.wave * 64);
    if (try_wave(wave, nl)) return;          // this lane was the last to arrive: everybody may go on
  }
  while (f->op != OP_NONE) yield_to_scheduler();
}

void run_block(dim3 grid, dim3 block, dim3 bid) {
  const int nt = (int)(block.x * block.y * block.z);
  if (nt > kMaxThreads) die("block of %d threads", nt);
  g_fibers.assign((size_t)nt, Fiber());
  while ((int)g_stacks.size() < nt) {
    void* p = mmap(nullptr, kStack, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS, -1, 0);
    if (p == MAP_FAILED) die("no memory for a fiber stack");
    mprotect(p, 4096, PROT_NONE);            // guard page under the stack
    g_stacks.push_back(static_cast<uint8_t*>(p));
  }
  g_uniform.assign((size_t)((nt + 63) / 64) * kUniformSlots, UniformTag{0, nullptr, 0, false});
  for (int t = 0; t < nt; ++t) {
    Fiber& f = g_fibers[t];
    f.lane.tid = dim3(t % block.x, (t / block.x) % block.y, t / (block.x * block.y));
    f.lane.bid = bid;
    f.lane.bdim = block;
    f.lane.gdim = grid;
    f.lane.lane = (unsigned)t & 63u;
    f.lane.wave = (unsigned)t >> 6;
    f.stack = g_stacks[t];
    uint64_t* top = reinterpret_cast<uint64_t*>(f.stack + kStack);
    *--top = 0;                               // keeps the entry frame aligned as after a call
    *--top = reinterpret_cast<uint64_t>(&fiber_main);
    for (int r = 0; r < 6; ++r) *--top = 0;
    f.sp = top;
  }
  int running = nt;
  const int nw = (nt + 63) / 64;
  while (running > 0) {
    bool progressed = false;
    // schedule 0: every wave advances by one rendezvous per sweep (the waves stay close together); 1 / 2: the
    // lowest / highest wave runs until it can go no further (a block barrier, its end) before the next one starts,
    // the largest skew between waves that the kernel's barriers allow
    for (int wi = 0; wi < nw; ++wi) {
      const int w = g_schedule == 2 ? nw - 1 - wi : wi;
      bool ran;
      do {
        ran = false;
        for (int t = w * 64; t < std::min(nt, w * 64 + 64); ++t) {
          Fiber& f = g_fibers[t];
          if (f.done || f.op != OP_NONE) continue;
          g_cur = &f;
          emu_switch(&g_sched_sp, f.sp);
          g_cur = nullptr;
          ran = progressed = true;
          if (f.done) --running;
        }
      } while (ran && g_schedule != 0);
    }
    if (running == 0) break;
    if (progressed) {
      bool any_runnable = false;
      for (int t = 0; t < nt; ++t) any_runnable = any_runnable || (!g_fibers[t].done && g_fibers[t].op == OP_NONE);
      if (any_runnable) continue;
    }
    // every running fiber waits.  Waves whose lanes all wait at one operation were served on arrival; what is left:
    // the block barrier (everybody at it), lanes that ended since (a wave's remaining lanes now agree), divergence.
    bool all_barrier = true;
    for (int t = 0; t < nt; ++t) all_barrier = all_barrier && (g_fibers[t].done || g_fibers[t].op == OP_BARRIER);
    if (all_barrier) {
      ++g_stat_rendezvous;
      for (int t = 0; t < nt; ++t) g_fibers[t].op = OP_NONE;
      continue;
    }
    bool served = false;
    for (int w = 0; w * 64 < nt && !served; ++w) served = try_wave(&g_fibers[w * 64], std::min(64, nt - w * 64));
    if (served) continue;
    // divergence: in some wave, serve the waiting group at the lowest code address
    for (int w = 0; w * 64 < nt && !served; ++w) {
      Fiber* wave = &g_fibers[w * 64];
      const int nl = std::min(64, nt - w * 64);
      const void* lowest = nullptr;
      for (int l = 0; l < nl; ++l)
        if (!wave[l].done && wave[l].op != OP_NONE && wave[l].op != OP_BARRIER && (lowest == nullptr || wave[l].site < lowest))
          lowest = wave[l].site;
      if (lowest == nullptr) continue;
      std::vector<int> who;
      for (int l = 0; l < nl; ++l)
        if (!wave[l].done && wave[l].site == lowest && wave[l].op != OP_NONE && wave[l].op != OP_BARRIER) who.push_back(l);
      perform(wave, who);
      served = true;
    }
    if (!served) die("deadlock: every fiber of block %u waits and nothing can be served", bid.x);
  }
}

uint8_t* lds_pointer(uint32_t lds32, unsigned bytes) {
  // kernels hold LDS addresses as 32-bit values; every LDS object of this emulation (function-local statics of the
  // kernels, g_dynamic_lds) lies in this shared object's data, whose upper address half g_dynamic_lds shares
  const uintptr_t hi = reinterpret_cast<uintptr_t>(g_dynamic_lds) & ~uintptr_t(0xffffffffu);
  uint8_t* p = reinterpret_cast<uint8_t*>(hi | lds32);
  const bool in_static = p >= __start_emu_lds && p + 64u * bytes <= __stop_emu_lds;
  const bool in_dynamic = p >= g_dynamic_lds && p < g_dynamic_lds + sizeof(g_dynamic_lds);
  if (!in_static && !in_dynamic) die("asynchronous load to %p, which is no LDS address", (void*)p);
  // a landing zone inside the dynamic LDS buffer must lie inside what the launch asked for
  if (p >= g_dynamic_lds && p < g_dynamic_lds + sizeof(g_dynamic_lds) &&
      (size_t)(p - g_dynamic_lds) + 64u * bytes > g_dynamic_bytes)
    die("asynchronous load lands at dynamic LDS offset %zu + %u bytes, the launch asked for %zu bytes",
        (size_t)(p - g_dynamic_lds), 64u * bytes, g_dynamic_bytes);
  return p;
}

}  // namespace

Lane& lane() { return g_cur->lane; }
uint8_t* dynamic_lds() { return g_dynamic_lds; }

void launch(dim3 grid, dim3 block, size_t dynamic_lds_bytes, const std::function<void()>& body) {
  emu_install_handlers();
  if (g_cur != nullptr) die("nested launch");
  if (dynamic_lds_bytes > sizeof(g_dynamic_lds)) die("%zu bytes of dynamic LDS", dynamic_lds_bytes);
  ++g_stat_launches;
  g_dynamic_bytes = dynamic_lds_bytes;
  g_body = &body;
  for (unsigned z = 0; z < grid.z; ++z)
    for (unsigned y = 0; y < grid.y; ++y)
      for (unsigned x = 0; x < grid.x; ++x) {
        ++g_stat_blocks;
        // a block finds no usable data in its LDS, dynamic or static: 0xFF bytes (NaN as e4m3, bf16 and fp32), so that a tile
        // the block forgot to load cannot pass as the previous block's copy of it
        memset(g_dynamic_lds, 0xFF, dynamic_lds_bytes);
        memset(__start_emu_lds, 0xFF, (size_t)(__stop_emu_lds - __start_emu_lds));
        run_block(grid, block, dim3(x, y, z));
      }
  g_body = nullptr;
}

void block_barrier() { rendezvous(OP_BARRIER, __builtin_return_address(0)); }
__attribute__((noinline)) void wave_sync() { rendezvous(OP_SYNC, __builtin_return_address(0)); }
__attribute__((noinline)) uint32_t shfl32(uint32_t v, int src) {
  g_cur->in[0] = v;
  g_cur->in[1] = (uint32_t)src;
  rendezvous(OP_SHFL, __builtin_return_address(0));
  return g_cur->out[0];
}
__attribute__((noinline)) uint32_t readlane32(uint32_t v, int l) {
  g_cur->in[0] = v;
  g_cur->in[1] = (uint32_t)l;
  rendezvous(OP_RLANE, __builtin_return_address(0));
  return g_cur->out[0];
}
__attribute__((noinline)) uint32_t update_dpp32(uint32_t old, uint32_t src, int ctrl, int row_mask, int bank_mask, bool bound_ctrl) {
  g_cur->in[0] = old;
  g_cur->in[1] = src;
  g_cur->in[2] = (uint32_t)ctrl;
  g_cur->in[3] = (uint32_t)row_mask;
  g_cur->in[4] = (uint32_t)bank_mask;
  g_cur->in[5] = bound_ctrl;
  rendezvous(OP_DPP, __builtin_return_address(0));
  return g_cur->out[0];
}
__attribute__((noinline)) uint64_t ballot(bool pred) {
  g_cur->in[0] = pred;
  rendezvous(OP_BALLOT, __builtin_return_address(0));
  return (uint64_t)g_cur->out[0] | ((uint64_t)g_cur->out[1] << 32);
}
__attribute__((noinline)) uint32_t readfirstlane32(uint32_t v) {
  g_cur->in[0] = v;
  rendezvous(OP_RFL, __builtin_return_address(0));
  return g_cur->out[0];
}
__attribute__((noinline)) void mfma_16x16x128_f8(const int32_t* a8, const int32_t* b8, const float* c4, float* d4) {
  memcpy(g_cur->in, a8, 32);
  memcpy(g_cur->in + 8, b8, 32);
  memcpy(g_cur->in + 16, c4, 16);
  rendezvous(OP_MFMA16_F8, __builtin_return_address(0));
  memcpy(d4, g_cur->out, 16);
}
__attribute__((noinline)) void mfma_32x32x64_f8(const int32_t* a8, const int32_t* b8, const float* c16, float* d16) {
  memcpy(g_cur->in, a8, 32);
  memcpy(g_cur->in + 8, b8, 32);
  memcpy(g_cur->in + 16, c16, 64);
  rendezvous(OP_MFMA32_F8, __builtin_return_address(0));
  memcpy(d16, g_cur->out, 64);
}
__attribute__((noinline)) void mfma_16x16x32_bf16(const uint16_t* a8, const uint16_t* b8, const float* c4, float* d4) {
  memcpy(g_cur->in, a8, 16);
  memcpy(g_cur->in + 4, b8, 16);
  memcpy(g_cur->in + 8, c4, 16);
  rendezvous(OP_MFMA16_BF16, __builtin_return_address(0));
  memcpy(d4, g_cur->out, 16);
}

void async_load(const void* base, uint32_t lane_off, uint32_t lds_base, unsigned bytes, bool uniform_base) {
  Fiber* f = g_cur;
  ++g_stat_async;
  // base and LDS address are scalar operands of the instruction: every lane of the wave must pass the same
  UniformTag& tag = g_uniform[(size_t)f->lane.wave * kUniformSlots + f->async_seq % kUniformSlots];
  const void* tag_base = uniform_base ? base : nullptr;       // (a per-lane address form has no scalar base)
  if (!tag.used || tag.seq != f->async_seq) tag = UniformTag{f->async_seq, tag_base, lds_base, true};
  else if (tag.base != tag_base || tag.lds != lds_base)
    die("asynchronous load %u of wave %u: lane %u passes another base or LDS address than an earlier lane", f->async_seq,
        f->lane.wave, f->lane.lane);
  ++f->async_seq;
  const uint8_t* src = static_cast<const uint8_t*>(base) + lane_off;
  uint8_t* dst = lds_pointer(lds_base, bytes) + (size_t)bytes * f->lane.lane;
  if (g_lazy) f->pending.push_back(Pending{src, dst, bytes});
  else memcpy(dst, src, bytes);
}

// An ordinary global load issued through the kernels' gload_* helpers: its value is delivered at once (the compiler
// places the wait for a register result itself), but under the counted lazy model it takes its place in the lane's
// queue of outstanding vector-memory operations, so that a wait_vm<N>() counts what the hardware counts.
void count_vm_load() {
  if (g_lazy && g_count_plain) g_cur->pending.push_back(Pending{nullptr, nullptr, 0});
}

void wait_vm(int n) {
  Fiber* f = g_cur;
  if (!g_lazy) return;
  const size_t keep = (size_t)(n <= 0 ? 0 : n + g_wait_slack);
  if (f->pending.size() <= keep) return;
  const size_t land = f->pending.size() - keep;
  for (size_t i = 0; i < land; ++i)
    if (f->pending[i].bytes) memcpy(f->pending[i].dst, f->pending[i].src, f->pending[i].bytes);
  f->pending.erase(f->pending.begin(), f->pending.begin() + (long)land);
}

float e4m3_to_f32(uint8_t b) {
  const int s = b >> 7, e = (b >> 3) & 15, m = b & 7;
  float v;
  if (e == 15 && m == 7) v = NAN;
  else if (e == 0) v = ldexpf((float)m, -9);
  else v = ldexpf((float)(8 + m), e - 10);
  return s ? -v : v;
}

// round to nearest even, saturating at +-448 (the library clamps before it converts), NaN -> 0x7f
uint8_t f32_to_e4m3(float f) {
  if (f != f) return 0x7f;
  const uint8_t sign = signbit(f) ? 0x80 : 0;
  float a = fabsf(f);
  if (a >= 448.0f) return sign | 0x7e;
  if (a < ldexpf(1.0f, -10)) return sign;                        // below half of the smallest denormal (2^-9)
  int e;
  (void)frexpf(a, &e);                                           // a = m 2^e, m in [0.5, 1)
  int exp = e - 1;                                               // a = 1.xxx 2^exp
  if (exp < -6) exp = -6;                                        // denormal range: fixed exponent
  const float q = rintf(ldexpf(a, 3 - exp));                     // mantissa in units of 2^(exp-3), ties to even
  int mant = (int)q, be = exp + 7;
  if (exp == -6 && mant < 8) return sign | (uint8_t)mant;        // denormal (or zero)
  if (mant == 16) { mant = 8; ++be; }
  if (be > 15 || (be == 15 && mant - 8 > 6)) return sign | 0x7e;
  return sign | (uint8_t)(be << 3) | (uint8_t)(mant - 8);
}

}  // namespace emu

#include <chrono>
double emu_now_ms() {
  using clock = std::chrono::steady_clock;
  return std::chrono::duration<double, std::milli>(clock::now().time_since_epoch()).count();
}

#include <execinfo.h>
#include <signal.h>
namespace {
void install_segv_handler();
struct Guarded { uint8_t* base; size_t map_bytes; uint8_t* data; size_t bytes; };
std::vector<Guarded> g_guarded;
void on_segv(int, siginfo_t* info, void*) {
  const uint8_t* a = static_cast<const uint8_t*>(info->si_addr);
  for (const Guarded& g : g_guarded)
    if (a >= g.base && a < g.base + g.map_bytes) {
      fprintf(stderr, "emu: access %ld bytes %s a guarded buffer of %zu bytes\n",
              a < g.data ? (long)(g.data - a) : (long)(a - (g.data + g.bytes)) + 1, a < g.data ? "in front of" : "past the end of",
              g.bytes);
      fflush(stderr);
      abort();
    }
  fprintf(stderr, "emu: segmentation fault at %p (not next to a guarded buffer%s)\n", (const void*)a,
          a == nullptr ? "; address 0 is also what a 16-byte access to a pointer that is not 16-byte aligned reports on x86" : "");
  if (emu::g_cur != nullptr)
    fprintf(stderr, "emu: in launch %llu, block %u, thread %u\n", (unsigned long long)emu::g_stat_launches,
            emu::g_cur->lane.bid.x, emu::g_cur->lane.tid.x);
  void* frames[24];
  const int n = backtrace(frames, 24);
  backtrace_symbols_fd(frames, n, 2);
  fflush(stderr);
  abort();
}
void install_segv_handler() {
  static bool handler = false;
  if (handler) return;
  static uint8_t alt[64 * 1024];
  stack_t ss;
  ss.ss_sp = alt; ss.ss_size = sizeof(alt); ss.ss_flags = 0;
  sigaltstack(&ss, nullptr);                      // a fiber that overran its stack has none left for the handler
  struct sigaction sa;
  memset(&sa, 0, sizeof(sa));
  sa.sa_sigaction = on_segv;
  sa.sa_flags = SA_SIGINFO | SA_ONSTACK;
  sigaction(SIGSEGV, &sa, nullptr);
  handler = true;
}
}  // namespace
void emu_install_handlers() { install_segv_handler(); }

extern "C" {
// A buffer whose last byte is the last byte of a page, with an inaccessible page behind it and another in front of its
// first page: an access past the end faults at once, and so does one more than a page's slack in front.  bytes is
// rounded up to a multiple of 16 (the slack lies at the front).
void* emu_guarded_alloc(size_t bytes) {
  install_segv_handler();
  const size_t page = 4096, padded = (bytes + 15) & ~size_t(15);
  const size_t body = (padded + page - 1) / page * page;
  uint8_t* base = static_cast<uint8_t*>(mmap(nullptr, body + 2 * page, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS, -1, 0));
  if (base == MAP_FAILED) return nullptr;
  mprotect(base, page, PROT_NONE);
  mprotect(base + page + body, page, PROT_NONE);
  uint8_t* data = base + page + body - padded;
  g_guarded.push_back(Guarded{base, body + 2 * page, data, padded});
  return data;
}
void emu_guarded_free(void* data) {
  for (size_t i = 0; i < g_guarded.size(); ++i)
    if (g_guarded[i].data == data) {
      munmap(g_guarded[i].base, g_guarded[i].map_bytes);
      g_guarded.erase(g_guarded.begin() + (long)i);
      return;
    }
}
void emu_set_wait_slack(int loads) { emu::g_wait_slack = loads < 0 ? 0 : loads; }
void emu_set_async_mode(int lazy) {                  // 0 eager, 1 lazy, 2 lazy with ordinary loads counted
  emu::g_lazy = lazy != 0;
  emu::g_count_plain = lazy == 2;
}
void emu_set_schedule(int mode) { emu::g_schedule = mode; }
void emu_stats(uint64_t* out4) {
  out4[0] = emu::g_stat_launches; out4[1] = emu::g_stat_blocks; out4[2] = emu::g_stat_rendezvous; out4[3] = emu::g_stat_async;
}
float emu_e4m3_to_f32(uint8_t b) { return emu::e4m3_to_f32(b); }
uint8_t emu_f32_to_e4m3(float f) { return emu::f32_to_e4m3(f); }
}
