// Instruction counts of the pipelined MFMA kernels' DMA side, and the s_waitcnt vmcnt(N) values derived from them:
// one definition for the kernels (gemm_mfma_pipe.hpp, gemm_mfma_pipe16.hpp) and for the host program that replays
// their issue order on the CPU and checks every count (tests/host_c/mfma_wait_check.cpp).
//
// The rule behind every N: the vector memory instructions of one wave that make a round trip to memory retire in the
// order they were issued, so "at most N outstanding" means "everything but the youngest N has landed".  An
// instruction whose lanes are ALL out of range makes no round trip and can retire ahead of older ones, so no kernel
// that counts issues one: padding stages and surplus scale instructions are real loads of one cache line, and an
// instruction of a K tail always holds the lane of its row's first chunk.  A wait that cannot be counted that way
// is vmcnt(0).
#pragma once

namespace zluda_amd {

struct PipeCounts {
  int cpr;      // 16-byte chunks per LDS row
  int rpw;      // rows filled by one wave DMA instruction
  int rpp;      // rows filled per DMA pass of the workgroup
  int lp, lq;   // data DMA instructions per thread, stage and operand
  int ndata;    // lp + lq
  int nwv;      // waves
  // MX block scales (zero without them): chunks of 32 scale bytes per tile row = ch stages, sparts instructions per
  // chunk, ls of them issued by every wave in front of every stage's data, pro_s per wave for the first chunk
  int sb, ch, sparts, ls, pro_s;
  int nload;    // ndata + ls: vector memory instructions per stage
  // Counted waits.  They count the DATA instructions of the younger stages only: the scale instructions of a stage
  // are issued in front of its data, so a wait that also covers them costs nothing.
  int wait_prologue;  // after the prologue (stages 0 .. nstage-1 issued): stage 0 has landed
  int wait_stage;     // in stage kt, before its slot is refilled: stage kt + 1 has landed
};

constexpr PipeCounts pipe_counts(bool mx, int bp, int bq, int wp, int wq, int bkb, int nstage) {
  PipeCounts c{};
  c.nwv = wp * wq;
  c.cpr = bkb / 16;
  c.rpw = 64 / c.cpr;
  c.rpp = c.nwv * c.rpw;
  c.lp = bp / c.rpp;
  c.lq = bq / c.rpp;
  c.ndata = c.lp + c.lq;
  c.sb = bkb / 16;
  c.ch = 32 / c.sb;
  c.sparts = (bp + bq) / 32;
  c.ls = mx ? (c.sparts + c.nwv * (c.ch - nstage) - 1) / (c.nwv * (c.ch - nstage)) : 0;
  c.pro_s = mx ? (c.sparts + c.nwv - 1) / c.nwv : 0;
  c.nload = c.ndata + c.ls;
  c.wait_prologue = (nstage - 1) * c.ndata;
  c.wait_stage = (nstage - 2) * c.ndata;
  return c;
}

// gemm_mfma_pipe16.hpp: two stages of 128 K bytes, eight rows per DMA instruction, no scale instructions
struct Pipe16Counts {
  int rpp, lp, lq, nload;
  int wait_prologue;  // stages 0 and 1 issued: stage 0 has landed
  int wait_stage;     // in stage kt, before its slot is refilled: stage kt + 1 has landed (nothing younger is in flight)
};

constexpr Pipe16Counts pipe16_counts(int bp, int bq, int wp, int wq) {
  Pipe16Counts c{};
  c.rpp = wp * wq * 8;
  c.lp = bp / c.rpp;
  c.lq = bq / c.rpp;
  c.nload = c.lp + c.lq;
  c.wait_prologue = c.nload;
  c.wait_stage = 0;
  return c;
}

// gemm_mfma_tr.hpp leaves its waits to the compiler, which counts: before the LDS stores of trip kt (stage kt + 1's
// registers) it waits until only stage kt + 2's loads are outstanding.  Stages hold 64 K bytes; only the last one that
// holds data, stage kl = ceil(kbytes / 64) - 1, can have lanes past the end of K (later trips load it again), and only
// when kbytes is no multiple of 64.  From the first trip whose younger stage is that one, the kernel waits for
// everything instead: the value below, compared with kt (0x7fffffff: never; negative: the prologue waits as well).
constexpr int tr_tail_from(int kbytes) {
  const int kt = (kbytes + 63) / 64, kl = kt > 0 ? kt - 1 : 0;
  return (kbytes & 63) ? kl - 2 : 0x7fffffff;
}

} // namespace zluda_amd
