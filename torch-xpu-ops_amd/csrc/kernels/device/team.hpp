// Device side of the exchange between the workgroups of a team (norm_fwd_team_kernel,
// softmax_fwd_team_kernel): a row too long for one workgroup is held in the registers of
// several, which pass two numbers each through library-owned device memory.  Below it: the
// same exchange in two halves for K float64 values (norm_fwd_rows_team_kernel, which puts
// a round of other work between publishing and gathering) and a lighter one of
// self-validating words for float32 values (norm_bwd_team_kernel).
//
// What crosses workgroups.  An entry is 128 bytes (neighbours' polls go to other memory
// channels).  The two-number exchange (team_publish_and_gather) uses {tag, s1, s2}: the tag
// of a finished entry is (call id << 32) | (round + 1), ids being unique per call, so nothing
// has to be cleared and an entry left by an earlier call or round never counts.  The writer
// sets the tag to 0 when it starts on a row, later stores s1 and s2, waits for those stores
// to be acknowledged and stores the tag; a reader accepts s1 and s2 only if it read the
// expected tag before and after them.  The exchanges in two halves further down write
// self-validating 64-bit words {32 bits of payload, tag} into the entry's pad[] instead: a
// word is valid or not by itself, so the writer orders nothing and waits for nothing and a
// reader needs one round trip (see team_publish_tagged).  Every access is a device-scope
// atomic store or load, which goes to memory: no read-modify-write (256 workgroups
// counting on one word took hundreds of microseconds), and no release or acquire fence
// (each writes back or invalidates a whole L2).  Two calls that were handed the same slot
// while both run -- possible only with more such calls in flight than slots -- overwrite
// each other's tags and therefore never accept each other's numbers.
//
// The wait is bounded, and no workgroup depends on another to finish.  A workgroup
// stops waiting when its team is complete, when any workgroup of the call has given
// up before (a hint word in the slot), or after `wait_ticks` of the constant-rate
// clock (the workgroups can only fail to be resident together while other kernels
// hold compute units for that long).  What a workgroup does without its team is the
// kernel's business; it keeps publishing its own numbers for the workgroups that do
// wait.
#pragma once

#include <stdint.h>

#include "../plan.hpp"
#include "reduce.hpp"

namespace rownorm {

__device__ __forceinline__ unsigned long long team_load(const unsigned long long* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void team_store(unsigned long long* p, unsigned long long v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Earlier stores of this lane have been acknowledged and its loads have returned.
__device__ __forceinline__ void team_stores_done() {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// team_word_tag: the tag every word of the exchanges below carries -- ((call id mod 2^25 - 1)
// + 1) << 6 | (round mod 64): never 0 (the memory starts as zeros), different for the rounds
// that share a buffer, different from call to call; bit 31 is clear.
//
// A workgroup that has stopped waiting for its team (`lost`) never publishes a valid word
// again: its words carry team_lost_tag -- the call's tag with bit 31 set, whatever the round
// -- and a gather that meets one gives up at once.  So the rest of its team follows it
// promptly, and -- tags repeat after 64 rounds -- nothing a workgroup writes while it runs
// ahead of its team on its own can be taken for the numbers of an earlier round.  The
// slot's hint word spreads the news to the other teams of the call, which look at it now
// and then.
__device__ __forceinline__ unsigned int team_word_tag(unsigned int call_id, unsigned int round) {
  return ((call_id % 0x1ffffffu) + 1u) << 6 | (round & 63u);
}
__device__ __forceinline__ unsigned int team_lost_tag(unsigned int call_id) {
  return 0x80000000u | team_word_tag(call_id, 0);
}
// (whether a word's tag is the call's lost tag)
__device__ __forceinline__ bool team_tag_is_lost(unsigned int tag, unsigned int call_id) {
  return (tag | 63u) == (team_lost_tag(call_id) | 63u);
}

// (A lane's entries are read four at a time: a round trip to memory for a team of up to 256,
// however many entries a lane has.)
constexpr int kTeamGatherBatch = 4;

// For the first wavefront of a workgroup (all 64 lanes, threadIdx.x < 64), whose entry
// `entries[blockIdx.x]` has had the tag 0 since the workgroup started on the row:
// publishes (a, b), waits for the `team` entries from `entries[tm * team]` on and leaves
// them in part[j][0..1] (LDS).  True when the team came together (the same in every lane);
// false after the wait ran out or another workgroup of the call gave up, which this one
// then records in the slot's hint word.
__device__ __forceinline__ bool team_publish_and_gather(TeamSlot* slot, TeamEntry* entries, int tm,
                                                        int team, unsigned int call_id,
                                                        unsigned int round,
                                                        unsigned long long wait_ticks, double a,
                                                        double b, double (*part)[2]) {
  const int lane = (int)threadIdx.x;
  const unsigned long long expect = ((unsigned long long)call_id << 32) | (round + 1u);
  if (lane == 0) {
    TeamEntry* mine = &entries[blockIdx.x];
    team_stores_done();  // the tag has been 0 in memory before the numbers change
    team_store(&mine->s1, __builtin_bit_cast(unsigned long long, a));
    team_store(&mine->s2, __builtin_bit_cast(unsigned long long, b));
    team_stores_done();
    team_store(&mine->tag, expect);
  }
  const TeamEntry* mates = entries + tm * team;
  const unsigned long long t0 = wall_clock64();
  bool complete = false;
  unsigned int polls = 0;
  for (;;) {
    bool ok = true;
    for (int j = lane; j < team; j += 64) ok = ok && team_load(&mates[j].tag) == expect;
    if (__ballot(ok) == __ballot(true)) {
      for (int j = lane; j < team; j += 64) {
        part[j][0] = __builtin_bit_cast(double, team_load(&mates[j].s1));
        part[j][1] = __builtin_bit_cast(double, team_load(&mates[j].s2));
        team_stores_done();  // the numbers have returned before the tag is read again
        ok = ok && team_load(&mates[j].tag) == expect;
      }
      if (__ballot(ok) == __ballot(true)) {
        complete = true;
        break;
      }
    }
    // (the hint word is one address for the whole grid: looked at every 16th time)
    if ((polls++ & 15u) == 0) {
      const unsigned int hint =
          __hip_atomic_load(&slot->gave_up, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (hint == call_id) break;
    }
    if (wall_clock64() - t0 > wait_ticks) break;
    __builtin_amdgcn_s_sleep(8);
  }
  if (lane == 0 && !complete)
    __hip_atomic_store(&slot->gave_up, call_id, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return complete;
}

// The exchange in two halves, for kernels that put other work between them; float32 values.
// Every 64-bit word carries its own tag, so a word is valid or not by itself and neither
// side orders anything.  Word k of an entry holds {v[k], tag}, tag = team_word_tag():
// different for the rounds that share a buffer (a buffer is reused every second or fourth
// round, and workgroups of a team whose gathers succeed are never more than three rounds
// apart), different from call to call.  The words live in an entry's pad[], which nothing
// else writes: whatever a word holds was put there by one of these exchanges.  Publishing
// is K plain stores with nothing to wait for; gathering reads every word of a lane's entries
// in one round trip and accepts them if every tag is the round's.  `lost`: see team_word_tag.
template <int K>
__device__ __forceinline__ void team_publish_tagged(TeamEntry* mine, unsigned int call_id,
                                                    unsigned int round, const float (&v)[K],
                                                    bool lost) {
  static_assert(K >= 1 && K <= 13, "an entry's pad[] holds 13 words");
  unsigned long long* words = &mine->pad[0];
  const unsigned long long tag =
      (unsigned long long)(lost ? team_lost_tag(call_id) : team_word_tag(call_id, round)) << 32;
#pragma unroll
  for (int k = 0; k < K; ++k)
    team_store(&words[k], tag | (unsigned long long)__builtin_bit_cast(unsigned int, v[k]));
}

// For the first wavefront of a workgroup (all 64 lanes).  On success v[] holds the sums over
// the team, added in a fixed order (entries lane, lane + 64, ... per lane, then across the
// lanes): the same bits in every lane and in every workgroup of the team.  False as in
// team_publish_and_gather; the workgroup publishes as `lost` from then on.
template <int K>
__device__ __forceinline__ bool team_gather_tagged(TeamSlot* slot, const TeamEntry* mates,
                                                   int team, unsigned int call_id,
                                                   unsigned int round,
                                                   unsigned long long wait_ticks, float (&v)[K]) {
  constexpr int B = kTeamGatherBatch;
  const int lane = (int)threadIdx.x;
  const unsigned int expect = team_word_tag(call_id, round);
  const unsigned long long t0 = wall_clock64();
  bool complete = false;
  unsigned int polls = 0;
  for (;;) {
    bool ok = true, lost_seen = false;
#pragma unroll
    for (int k = 0; k < K; ++k) v[k] = 0.0f;
    for (int j0 = lane; j0 < team; j0 += 64 * B) {
      unsigned long long w[B][K];
#pragma unroll
      for (int b = 0; b < B; ++b) {
        const int j = j0 + 64 * b;
#pragma unroll
        for (int k = 0; k < K; ++k) w[b][k] = 0;
        if (j < team) {
          const unsigned long long* words = &mates[j].pad[0];
#pragma unroll
          for (int k = 0; k < K; ++k) w[b][k] = team_load(&words[k]);
        }
      }
#pragma unroll
      for (int b = 0; b < B; ++b) {
        if (j0 + 64 * b < team) {
#pragma unroll
          for (int k = 0; k < K; ++k) {
            ok = ok && (unsigned int)(w[b][k] >> 32) == expect;
            lost_seen = lost_seen || team_tag_is_lost((unsigned int)(w[b][k] >> 32), call_id);
            v[k] += __builtin_bit_cast(float, (unsigned int)(w[b][k] & 0xffffffffull));
          }
        }
      }
    }
    if (__ballot(lost_seen) != 0) break;
    if (__ballot(ok) == __ballot(true)) {
#pragma unroll
      for (int k = 0; k < K; ++k) v[k] = wave_group_allreduce<64, SumOp>(v[k]);
      complete = true;
      break;
    }
    // (the hint word is one address for the whole grid: looked at every 16th time)
    if ((polls++ & 15u) == 0) {
      const unsigned int hint =
          __hip_atomic_load(&slot->gave_up, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (hint == call_id) break;
    }
    if (wall_clock64() - t0 > wait_ticks) break;
    __builtin_amdgcn_s_sleep(8);
  }
  if (!complete && lane == 0)
    __hip_atomic_store(&slot->gave_up, call_id, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return complete;
}

// The same two halves for K float64 values a workgroup (K <= 6), each cut into two words
// {32 bits, tag} of pad[] as in team_publish_and_gather, summed over the team in the fixed
// order of team_gather_tagged.
template <int K>
__device__ __forceinline__ void team_publish_f64(TeamEntry* mine, unsigned int call_id,
                                                 unsigned int round, const double (&v)[K],
                                                 bool lost) {
  static_assert(K >= 1 && 2 * K <= 13, "an entry's pad[] holds 13 words");
  unsigned long long* words = &mine->pad[0];
  const unsigned long long tag =
      (unsigned long long)(lost ? team_lost_tag(call_id) : team_word_tag(call_id, round)) << 32;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const unsigned long long bits = __builtin_bit_cast(unsigned long long, v[k]);
    team_store(&words[2 * k], tag | (bits & 0xffffffffull));
    team_store(&words[2 * k + 1], tag | (bits >> 32));
  }
}

template <int K>
__device__ __forceinline__ bool team_gather_sums_f64(TeamSlot* slot, const TeamEntry* mates,
                                                     int team, unsigned int call_id,
                                                     unsigned int round,
                                                     unsigned long long wait_ticks,
                                                     double (&v)[K]) {
  constexpr int B = kTeamGatherBatch;
  const int lane = (int)threadIdx.x;
  const unsigned int expect = team_word_tag(call_id, round);
  const unsigned long long t0 = wall_clock64();
  bool complete = false;
  unsigned int polls = 0;
  for (;;) {
    bool ok = true, lost_seen = false;
#pragma unroll
    for (int k = 0; k < K; ++k) v[k] = 0.0;
    for (int j0 = lane; j0 < team; j0 += 64 * B) {
      unsigned long long w[B][2 * K];
#pragma unroll
      for (int b = 0; b < B; ++b) {
        const int j = j0 + 64 * b;
#pragma unroll
        for (int k = 0; k < 2 * K; ++k) w[b][k] = 0;
        if (j < team) {
          const unsigned long long* words = &mates[j].pad[0];
#pragma unroll
          for (int k = 0; k < 2 * K; ++k) w[b][k] = team_load(&words[k]);
        }
      }
#pragma unroll
      for (int b = 0; b < B; ++b) {
        if (j0 + 64 * b < team) {
#pragma unroll
          for (int k = 0; k < K; ++k) {
            ok = ok && (unsigned int)(w[b][2 * k] >> 32) == expect &&
                 (unsigned int)(w[b][2 * k + 1] >> 32) == expect;
            lost_seen = lost_seen || team_tag_is_lost((unsigned int)(w[b][2 * k] >> 32), call_id);
            v[k] += __builtin_bit_cast(double,
                                       (w[b][2 * k] & 0xffffffffull) | (w[b][2 * k + 1] << 32));
          }
        }
      }
    }
    if (__ballot(lost_seen) != 0) break;
    if (__ballot(ok) == __ballot(true)) {
#pragma unroll
      for (int k = 0; k < K; ++k) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) v[k] += __shfl_xor(v[k], off, 64);
      }
      complete = true;
      break;
    }
    // (the hint word is one address for the whole grid: looked at every 16th time)
    if ((polls++ & 15u) == 0) {
      const unsigned int hint =
          __hip_atomic_load(&slot->gave_up, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (hint == call_id) break;
    }
    if (wall_clock64() - t0 > wait_ticks) break;
    __builtin_amdgcn_s_sleep(8);
  }
  if (!complete && lane == 0)
    __hip_atomic_store(&slot->gave_up, call_id, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return complete;
}

}  // namespace rownorm
