// CPU emulator for the kernels' execution model: test infrastructure only, never part of the
// product.  One OS thread runs a workgroup's lanes as cooperative fibers; operations that involve
// a whole wavefront (cross-lane moves, ballots, matrix instructions, transposing LDS reads) and
// workgroup barriers are rendezvous points.  Workgroups of a launch run one after another.
//
// What it models beyond plain arithmetic:
//   * wave64 lane semantics of every cross-lane operation the kernels use,
//   * register layouts of the MFMA instructions and of ds_read_b64_tr_b16,
//   * LDS as one arena addressed by 32-bit addresses, trashed before every workgroup,
//   * global -> LDS moves that complete late (at the wait) or early (at issue), selectable,
//     so that both a missing wait and a slot overwritten too soon change the results,
//   * a collective reached by only part of a wavefront's live lanes aborts with a message.
#pragma once
#include <stddef.h>
#include <stdint.h>

#include <functional>

namespace emu {

struct Dim3 {
  unsigned x, y, z;
  constexpr Dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};

constexpr int kWave = 64;
constexpr int kSlotBytes = 128;        // operand bytes a lane can post per collective

struct Wave;
struct Lane {
  Dim3 tid;
  int lane;                            // lane id in its wavefront
  int flat;                            // thread id in the workgroup
  Wave* wave;
  int parity = 0;                      // slot set of the last rendezvous this lane went through
};

Lane* self();                          // the lane that is running now
Dim3 block_idx();
Dim3 block_dim();
Dim3 grid_dim();

// Rendezvous of the live lanes of the calling lane's wavefront.  `tag` names the operation; lanes
// arriving with different tags (divergent control flow around a collective) abort the process.
// Returns the parity of the slot set posted for this rendezvous.
int wave_rendezvous(const void* post, size_t bytes, uint32_t tag);
const uint8_t* wave_slot(int parity, int lane);      // what `lane` posted (valid until the next rendezvous but one)
bool wave_lane_live(int lane);                       // `lane` took part in the calling lane's last rendezvous
void block_barrier();
void poll_yield();                                   // inside a loop that polls memory another workgroup writes: lets the others run

// LDS arena: every __shared__ object lives in the ELF section "emu_lds"
uint32_t lds_addr(const void* p);
uint8_t* lds_ptr(uint32_t addr, size_t bytes);       // bounds-checked

// global -> LDS moves
void dma_issue(const void* src, uint32_t lds_dst, int bytes);
void dma_wait(int allowed_in_flight);

// LDS bank accounting (off unless emu_set_lds_profile(1)): a wavefront-wide LDS access by 32-bit
// address, `bytes` per lane, is a rendezvous of the wavefront; the access is priced as the hardware
// serves it: 16-byte accesses 16 lanes at a time, 8-byte accesses 32 lanes at a time, 64 banks of
// 4 bytes, one pass per distinct word a bank is asked for.  kind: 0 read, 1 transposing read, 2 write.
void lds_account(uint32_t addr, int bytes, int kind);
// Work counters (always on, cheap): per-lane calls scaled to wavefront instructions by the caller.
void count_mfma(int m, int k);                        // one lane's share of a wavefront MFMA: M x M x K
struct WorkCounts {
  unsigned long long mfma_lane_calls, mfma_flops, lds_read_bytes, lds_write_bytes, dma_bytes, dma_lane_calls, barriers_lane_calls;
};
extern WorkCounts g_work;

void launch(Dim3 grid, Dim3 block, const std::function<void()>& body);
int cu_count();                       // what the stand-in device reports as its number of compute units

[[noreturn]] void fail(const char* fmt, ...);

}  // namespace emu

extern "C" {
// knobs for the tests
void emu_set_dma_mode(int eager);        // 0: moves land at the wait (default), 1: at issue
void emu_set_block_order(unsigned seed); // 0: ascending block ids, else a seeded shuffle
void emu_set_wave_skew(unsigned seed);   // 0: a workgroup's wavefronts advance together; else they run one at a time for random
                                         // stretches; from 1000 on wavefront (seed % wavefronts) also moves only when no other can
// n > 1: up to n workgroups share the machine, each advancing a few scheduling steps at a time in a seeded random order
// (a workgroup that polls for another one's writes then really waits); else one workgroup after the other
void emu_set_concurrent_blocks(unsigned n, unsigned seed);
unsigned long long emu_launch_count(void);
unsigned long long emu_block_count(void);  // workgroups of all launches since the library was loaded
unsigned long long emu_poll_count(void);  // times a lane gave way inside a polling loop since the library was loaded
void emu_set_cu_count(int n);            // before the library's first query (it caches the answer); default 256
void emu_set_lds_profile(int on);        // 1: count bank passes of the kernels' addressed LDS accesses (slower); resets the counts
// out[3 * kind + 0] wavefront instructions, + 1 passes they took, + 2 passes a conflict-free access would take
void emu_lds_profile(unsigned long long out[9]);
// out: MFMA wavefront instructions, MFMA flops, addressed LDS bytes read, written, global -> LDS bytes moved,
// move wavefront instructions (a partly filled one counts by its active lanes / 64), workgroup barriers x wavefronts
void emu_work_counts(double out[7], int reset);
}
