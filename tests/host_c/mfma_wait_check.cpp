// Host-side replay of the DMA issue order of the pipelined MFMA kernels, with the kernels' own instruction counts and
// wait values (zluda_amd/csrc/kernels/mfma_wait_counts.hpp) and the planner's table of instantiated tile variants:
// at every counted s_waitcnt vmcnt(N) of every variant
//   * the stage the wait is there for has landed, given that a wave's loads retire in the order they were issued,
//   * N is exactly the number of DATA instructions issued after that stage's last one (one more would let the wait pass
//     early, one less would wait for a stage that should stay in flight),
//   * the MX scale chunk a stage reads landed before the barrier in front of the read.
// For the transposing kernel, which leaves the counting to the compiler: every trip whose younger stage in flight can
// hold lanes past the end of K is one that waits for everything.
// usage: mfma_wait_check   (prints the number of waits checked, exits non-zero on the first violation)
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../../zluda_amd/csrc/kernels/mfma_wait_counts.hpp"
#include "../../zluda_amd/csrc/planner.hpp"

using namespace zluda_amd;

enum { DATA, SCALE, SURPLUS };
struct Ins { int kind, id; };  // DATA: stage; SCALE: chunk; SURPLUS: -

static long checked = 0;

static void fail(const char *what, int variant, int mx, int wave, int kt, int KT) {
  printf("variant %d mx %d wave %d stage %d of %d: %s\n", variant, mx, wave, kt, KT, what);
  exit(1);
}

// the youngest `n` of `log` are outstanding: has every instruction of (kind, id) landed?
static bool landed(const std::vector<Ins> &log, size_t issued, int n, int kind, int id) {
  for (size_t i = issued > (size_t)n ? issued - n : 0; i < issued; i++)
    if (log[i].kind == kind && log[i].id == id) return false;
  return true;
}
// DATA instructions issued after the last one of `stage`
static int data_after(const std::vector<Ins> &log, int stage) {
  int last = -1;
  for (size_t i = 0; i < log.size(); i++)
    if (log[i].kind == DATA && log[i].id == stage) last = (int)i;
  if (last < 0) return -1;
  int n = 0;
  for (size_t i = last + 1; i < log.size(); i++) n += log[i].kind == DATA;
  return n;
}

// gemm_mfma_pipe_kernel: prologue, then per stage [reads of the next stage's scales] wait, barrier, scale instructions,
// data of stage kt + nstage
static void check_pipe(int variant, bool mx, int ks) {
  const MfmaVariant &v = kMfmaVariants[variant];
  const PipeCounts c = pipe_counts(mx, v.bp, v.bq, v.wp, v.wq, v.bkb, v.stages);
  if ((v.stages - 1) * c.nload >= 64) fail("vmcnt range", variant, mx, 0, 0, 0);
  for (int KT = 1; KT <= 3 * c.ch + v.stages + 2; KT++)
    for (int wave = 0; wave < c.nwv; wave++) {
      std::vector<Ins> log;
      auto scale_part = [&](int chunk, int part) { log.push_back(part < c.sparts ? Ins{SCALE, chunk} : Ins{SURPLUS, 0}); };
      auto data = [&](int stage) { for (int i = 0; i < c.ndata; i++) log.push_back(Ins{DATA, stage}); };
      for (int i = 0; i < c.pro_s; i++) scale_part(0, i * c.nwv + wave);
      for (int s = 0; s < v.stages; s++) {
        for (int i = 0; i < c.ls; i++) scale_part(0, c.sparts);
        data(s);
      }
      size_t wait_at = log.size();  // instructions issued at the last wait, and its N
      int wait_n = c.wait_prologue;
      if (!landed(log, wait_at, wait_n, DATA, 0)) fail("prologue: stage 0 still in flight", variant, mx, wave, 0, KT);
      if (data_after(log, 0) != wait_n) fail("prologue: N is not the count of younger data instructions", variant, mx, wave, 0, KT);
      if (mx && !landed(log, wait_at, wait_n, SCALE, 0)) fail("prologue: first scale chunk still in flight", variant, mx, wave, 0, KT);
      checked++;
      for (int kt = 0; kt < KT; kt++) {
        const int next_chunk = (kt + 1) / c.ch;
        // several sub-steps: the scales of stage kt + 1 are read in the first one, under the previous barrier
        if (mx && ks > 1 && kt + 1 < KT && !landed(log, wait_at, wait_n, SCALE, next_chunk))
          fail("scale chunk read before it landed", variant, mx, wave, kt, KT);
        wait_at = log.size();
        wait_n = c.wait_stage;
        if (!landed(log, wait_at, wait_n, DATA, kt + 1)) fail("next stage still in flight", variant, mx, wave, kt, KT);
        if (data_after(log, kt + 1) != wait_n) fail("N is not the count of younger data instructions", variant, mx, wave, kt, KT);
        if (mx && ks == 1 && kt + 1 < KT && !landed(log, wait_at, wait_n, SCALE, next_chunk))
          fail("scale chunk read before it landed", variant, mx, wave, kt, KT);
        checked++;
        for (int i = 0; i < c.ls; i++) scale_part(kt / c.ch + 1, ((kt % c.ch) * c.ls + i) * c.nwv + wave);
        data(kt + v.stages);
      }
      // every part of every chunk that a stage reads was issued by some wave: parts [0, sparts) over the waves
      if (mx && wave == 0) {
        std::vector<int> seen(c.sparts, 0);
        for (int w = 0; w < c.nwv; w++)
          for (int kt = 0; kt < c.ch; kt++)
            for (int i = 0; i < c.ls; i++) {
              const int part = ((kt % c.ch) * c.ls + i) * c.nwv + w;
              if (part < c.sparts) {
                if (kt >= c.ch - v.stages) fail("a scale part is issued too late in its chunk", variant, mx, w, kt, KT);
                seen[part]++;
              }
            }
        for (int p = 0; p < c.sparts; p++)
          if (seen[p] != 1) fail("scale parts of a chunk not issued exactly once", variant, mx, 0, p, KT);
      }
    }
}

// gemm_mfma_pipe16_kernel: stages 0 and 1, wait; per stage wait, barrier, data of stage kt + 2
static void check_pipe16(int variant) {
  const MfmaVariant &v = kMfmaVariants[variant];
  const Pipe16Counts c = pipe16_counts(v.bp, v.bq, v.wp, v.wq);
  if (v.stages != 2 || v.bkb != 128) fail("two stages of 128 bytes", variant, 0, 0, 0, 0);
  for (int KT = 1; KT <= 9; KT++) {
    std::vector<Ins> log;
    auto data = [&](int stage) { for (int i = 0; i < c.nload; i++) log.push_back(Ins{DATA, stage}); };
    data(0); data(1);
    if (!landed(log, log.size(), c.wait_prologue, DATA, 0)) fail("prologue: stage 0 still in flight", variant, 0, 0, 0, KT);
    if (data_after(log, 0) != c.wait_prologue) fail("prologue: N is not the count of younger data instructions", variant, 0, 0, 0, KT);
    checked++;
    for (int kt = 0; kt < KT; kt++) {
      if (!landed(log, log.size(), c.wait_stage, DATA, kt + 1)) fail("next stage still in flight", variant, 0, 0, kt, KT);
      if (data_after(log, kt + 1) != c.wait_stage) fail("N is not the count of younger data instructions", variant, 0, 0, kt, KT);
      checked++;
      data(kt + 2);
    }
  }
}

// gemm_mfma_tr_kernel: trip kt stores stage kt + 1's registers while stage min(kt + 2, kl)'s loads are in flight
static void check_tr() {
  for (int kbytes = 1; kbytes <= 64 * 9; kbytes++) {
    const int KT = (kbytes + 63) / 64, KL = KT > 0 ? KT - 1 : 0;
    const int tail_from = tr_tail_from(kbytes);
    auto may_hold_lanes_past_k = [&](int stage) { return stage >= KL && (kbytes & 63) != 0; };
    // the prologue stores stage 0 with the loads of stage min(1, KL) in flight
    if (may_hold_lanes_past_k(1 < KL ? 1 : KL) && !(tail_from < 0)) {
      printf("transposing kernel, K = %d bytes: the prologue counts past a stage that can retire early\n", kbytes);
      exit(1);
    }
    for (int kt = 0; kt + 1 <= KL; kt++) {  // trips that still store a stage
      const int younger = kt + 2 < KL ? kt + 2 : KL;
      if (may_hold_lanes_past_k(younger) && !(kt >= tail_from)) {
        printf("transposing kernel, K = %d bytes, trip %d: counts past a stage that can retire early\n", kbytes, kt);
        exit(1);
      }
      checked++;
    }
    if ((kbytes & 63) == 0 && tail_from != 0x7fffffff) { printf("transposing kernel, K = %d bytes: needless waits\n", kbytes); exit(1); }
  }
}

int main() {
  for (int variant = 0; variant < kNumMfmaVariants; variant++) {
    const MfmaVariant &v = kMfmaVariants[variant];
    if (v.w4) continue;  // every wait of the four-wave kernel is vmcnt(0) (checked on its source)
    if (v.m16) { check_pipe16(variant); continue; }
    // sub-steps per stage: 32 K bytes each, fp8 64; with and without MX scales where the variant serves MXFP4
    for (int ks : {v.bkb / 32, v.bkb / 64}) check_pipe(variant, false, ks);
    if (variant < kNumMfmaVariants32) check_pipe(variant, true, v.bkb / 32);
  }
  check_tr();
  printf("%ld waits checked\n", checked);
  return 0;
}
