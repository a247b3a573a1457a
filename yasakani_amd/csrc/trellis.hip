// Trellis-coded KV rows (the reference's KV4 / KV5 row formats) on gfx950: encoder, packing, decoder.
//   reference: src/kvq_gpu.cuh:51-147 (one row per block), src/kvq_fast.cuh:63-233 (production: a block per
//   row x multiplier x chunk, then a select-and-pack block per row), decode src/kvq_attn.cuh:46-75.
// Every fp32 value is produced by the same sequence of single IEEE operations as there (explicit __f*_rn calls, sums in
// the reference's order: inside each run of 32 elements the butterfly a[i] += a[i ^ o], o = 16 .. 1, then the 8 run sums
// added in order), and the path search works on integers with the reference's tie rules, so rows are bit-identical.
//
// How the search is laid out is specific to wave64: a chunk of 64 elements is one path through 256 states and belongs to
// ONE wave, four states per lane.  The states that can precede state d are the group { p : p mod U == d >> kk } (U =
// 256 >> kk), so a step is "minimum of every group, then add each state's own step cost".  For 4- and 5-bit fields the
// costs alternate between two lane arrangements chosen so that a group's minimum, found by lane-crossing minimum
// instructions (quad permutations, row rotations, the row / half swaps of gfx950), already sits in the lanes whose states
// continue that group: no barrier, no cost array in LDS, no LDS round trip.  Cost and predecessor index travel in one
// 32-bit key, so one reduction yields both and the reference's tie rule (smallest predecessor); the step cost
// (x - c)^2 loses the x^2 common to all states and becomes one 24-bit multiply-add.  The chosen predecessors (one per
// group and step) go to a 2 KB LDS block private to the wave, a word per four steps, and are walked back in parallel
// blocks.  3-bit fields keep a plainer form (group minima gathered through LDS, one lane walks back).
#include "yka_internal.h"
#include "rot256_device.h"
#include <hip/hip_fp16.h>

namespace yka {
namespace {

// ---- the profile blob, read where it lies (little-endian, no alignment assumed) ----
// The encoder kernels also get what the host has already looked up in the blob (`desc`, see TbEncArgs): one aligned
// 32-byte record per group and the tables as aligned int16, so that a block reaches its table after ONE dependent load
// instead of four (header -> offset of the group record -> record -> offset of the table record -> table).
struct Profile {
  const uint8_t* base;
  const uint32_t* desc = nullptr; int n_groups = 0; unsigned mult_off = 0;
  __device__ unsigned half_at(unsigned off) const { return base[off] | ((unsigned)base[off + 1] << 8); }
  __device__ unsigned word_at(unsigned off) const { return half_at(off) | (half_at(off + 2) << 16); }
  __device__ float float_at(unsigned off) const { return __uint_as_float(word_at(off)); }
  __device__ float f16_at(unsigned off) const { return __half2float(__ushort_as_half((unsigned short)half_at(off))); }
  __device__ unsigned groups() const { return desc ? (unsigned)n_groups : word_at(28); }
  __device__ float multiplier(int i) const { return float_at((desc ? mult_off : word_at(32)) + 4u * (unsigned)i); }
  __device__ unsigned table_record(int t) const { return word_at(word_at(36) + 4u * (unsigned)t); }
  __device__ unsigned group_record(int g) const { return word_at(word_at(40) + 4u * (unsigned)g); }
};
// what a group record says; `present` is false for a group index the profile does not have
struct GroupRec {
  bool present; int mode, bits, table, guard, ndir; bool has_mean;
  unsigned mean_off, dir_off;            // byte offsets of the fp16 mean row and of the first fp16 direction
  const int16_t* ints; float gain;       // descriptor form: the group's table
};
__device__ __forceinline__ GroupRec read_group(const Profile& P, int g) {
  GroupRec G{};
  G.present = (unsigned)g < P.groups();
  G.bits = 4;
  if (!G.present) return G;
  if (P.desc) {
    const uint4 lo = *reinterpret_cast<const uint4*>(P.desc + 8 * (size_t)g);
    const uint2 hi = *reinterpret_cast<const uint2*>(P.desc + 8 * (size_t)g + 4);
    G.mode = lo.x & 255u; G.bits = (lo.x >> 8) & 255u; G.table = (lo.x >> 16) & 255u; G.guard = lo.x >> 24;
    G.ndir = lo.y & 255u; G.has_mean = (lo.y >> 8) != 0u;
    G.mean_off = lo.z; G.dir_off = lo.w;
    G.ints = reinterpret_cast<const int16_t*>(P.desc) + hi.x; G.gain = __uint_as_float(hi.y);
    return G;
  }
  const unsigned rec = P.group_record(g);
  G.mode = P.base[rec]; G.bits = P.base[rec + 1]; G.table = P.base[rec + 2]; G.guard = P.base[rec + 3];
  G.ndir = P.base[rec + 4]; G.has_mean = P.base[rec + 5] != 0;
  G.mean_off = rec + 8; G.dir_off = G.mean_off + (G.has_mean ? 512u : 0u);
  return G;
}
// table of a trellis group: value of state s = (int16 at values + 2 s) / 256 * gain, each product rounded to fp32
struct TableRec { unsigned values; float gain; const int16_t* ints; };
__device__ __forceinline__ TableRec read_table(const Profile& P, const GroupRec& G) {
  if (G.ints) return TableRec{0u, G.gain, G.ints};
  const unsigned rec = P.table_record(G.table);
  return TableRec{rec + 12u, P.float_at(rec + 4u), nullptr};
}
__device__ __forceinline__ int table_int(const Profile& P, const TableRec& T, int state) {
  return T.ints ? (int)T.ints[state] : (int)(short)P.half_at(T.values + 2u * (unsigned)state);
}
__device__ __forceinline__ float table_value(int ti, float gain) { return __fmul_rn(__fmul_rn((float)ti, 1.f / 256.f), gain); }

// fp32 value -> nearest fp16 -> fp32.  The empty asm keeps the compiler from merging the operation that produced v with the
// conversion into one mixed-precision instruction, which would skip the fp32 rounding the reference performs in between
__device__ __forceinline__ float round_f16(float v) { asm volatile("" : "+v"(v)); return __half2float(__float2half_rn(v)); }

// Reduction over the 256 threads of a block in the order the reference fixes (src/kvq_fast.cuh:31-52): inside each run of
// 32 elements the butterfly a[i] = op(a[i], a[i ^ o]), o = 16 .. 1, then the 8 run results folded in order from `start`.
struct AddRn { __device__ static float op(float a, float b) { return __fadd_rn(a, b); } };
struct MaxOp { __device__ static float op(float a, float b) { return fmaxf(a, b); } };
template <class Op>
__device__ __forceinline__ float block_fold(float* part8, float v, float start) {
#pragma unroll
  for (int o = 16; o; o >>= 1) v = Op::op(v, __shfl_xor(v, o, 64));         // partners stay inside a half of the wave
  const int run = threadIdx.x >> 5;
  if ((threadIdx.x & 31) == 0) part8[run] = v;
  __syncthreads();
  float acc = start;
#pragma unroll
  for (int k = 0; k < 8; ++k) acc = Op::op(acc, part8[k]);
  __syncthreads();
  return acc;
}

// ---- which row a block works on ----
struct RowRef {
  float x;             // element threadIdx.x of the row (after the optional rotation)
  int group, pos;      // profile group and position
  size_t index;        // probe form: the row's index in the arrays; cache form: kv head * max_ctx + position
  int is_v;            // cache form: 0 K row, 1 V row
  size_t container;    // cache form, multi-stream pass: byte offset of the row's container
  bool valid;          // multi-stream pass: false if the row names no container
};
// Probe form: rows with their own group and position.  Cache form: row r of the launch = (token r / (2 n_kv), K | V, kv head)
__device__ __forceinline__ RowRef locate_row(const TbEncArgs& A, int r, float* rot_buf) {
  const int d = threadIdx.x;
  RowRef R{};
  R.valid = true;
  if (A.yin) {
    R.index = (size_t)(A.row0 + r);
    R.group = A.grp[R.index]; R.pos = A.pos[R.index]; R.x = A.yin[R.index * 256 + d];
  } else {
    const int per_tok = 2 * A.n_kv, tok = A.tok0 + r / per_tok, within = r % per_tok;
    R.is_v = within / A.n_kv;
    const int kvh = within % A.n_kv;
    if (A.rows.pos) {                                  // multi-stream pass: the row's own container and position
      const int slot = A.rows.slot[tok];
      R.pos = A.rows.pos[tok];
      R.valid = slot >= 0 && slot < A.rows.n_slots;
      R.container = R.valid ? (size_t)slot * A.rows.slot_bytes : 0;
    } else {
      R.pos = *A.d_pos + tok;
    }
    R.group = (A.layer * A.n_kv + kvh) * 2 + R.is_v;
    const size_t src = ((size_t)tok * A.n_kv + kvh) * 256 + d;
    R.x = A.k32 ? (R.is_v ? A.v32 : A.k32)[src] : __half2float(__ushort_as_half((R.is_v ? A.v16 : A.k16)[src]));
    R.index = (size_t)kvh * A.max_ctx + (size_t)max(0, min(R.pos, A.max_ctx - 1));
  }
  if (A.rot) R.x = rotate256(R.x, rot_buf, false);
  return R;
}

// ---- the step before coding (src/kvq_fast.cuh:63-76): remove the mean row, project out up to two directions with
//      coefficients rounded to fp16, measure the rms of what is left ----
struct Residual { float r, mean, coef[2], dir[2], rms; };
__device__ __forceinline__ Residual residual_of(float* part8, const Profile& P, const GroupRec& G, float x) {
  const unsigned d = threadIdx.x;
  Residual Q{};
  Q.r = x;
  if (G.has_mean) { Q.mean = P.f16_at(G.mean_off + 2u * d); Q.r = __fsub_rn(x, Q.mean); }
#pragma unroll
  for (int k = 0; k < 2; ++k) {                        // at most two directions; the test is uniform over the block (barriers inside)
    if (k >= G.ndir) break;
    Q.dir[k] = P.f16_at(G.dir_off + 512u * (unsigned)k + 2u * d);
    Q.coef[k] = round_f16(block_fold<AddRn>(part8, __fmul_rn(Q.r, Q.dir[k]), 0.f));
    Q.r = __fsub_rn(Q.r, __fmul_rn(Q.coef[k], Q.dir[k]));
  }
  const float mean_sq = __fdiv_rn(block_fold<AddRn>(part8, __fmul_rn(Q.r, Q.r), 0.f), 256.f);
  Q.rms = sqrtf(mean_sq);                              // sqrtf is correctly rounded on this target
  if (Q.rms == 0.f) Q.rms = 1.f;
  return Q;
}
// scale tried for a multiplier: rms * multiplier rounded to fp32, then to fp16; 0 -> 1
__device__ __forceinline__ float trial_scale(float rms, float multiplier) {
  const float s = round_f16(__fmul_rn(rms, multiplier));
  return s == 0.f ? 1.f : s;
}

// min over the lane pair (l, l ^ O) without an LDS round trip: a row rotation for O = 8, the gfx950 row / half swaps for
// O = 16 and 32 (after swapping a register with a copy of itself the two results hold, in every lane, the values of the
// lane and of its partner)
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
template <int O>
__device__ __forceinline__ int pair_min(int v) {
  if constexpr (O == 8) return min(v, __builtin_amdgcn_update_dpp(v, v, 0x128, 0xf, 0xf, false));      // row_ror:8
  else if constexpr (O == 16) { const u32x2 r = __builtin_amdgcn_permlane16_swap((unsigned)v, (unsigned)v, false, false); return min((int)r[0], (int)r[1]); }
  else { const u32x2 r = __builtin_amdgcn_permlane32_swap((unsigned)v, (unsigned)v, false, false); return min((int)r[0], (int)r[1]); }
}
template <int U>
__device__ __forceinline__ int group_min(int v) {       // min over the lanes congruent modulo U (U = 8, 16, 32)
  if constexpr (U <= 8) v = pair_min<8>(v);
  if constexpr (U <= 16) v = pair_min<16>(v);
  return pair_min<32>(v);
}

// min(v, v of the lane a DPP control names) as ONE instruction.  The compiler's own form is copy + move-with-control +
// min; the two idle cycles a lane-crossing read needs after its source was written are part of the statement.
#define YKA_DPP_MIN(NAME, CTRL)                                                                                  \
  __device__ __forceinline__ int NAME(int v) {                                                                   \
    int r;                                                                                                       \
    asm("s_nop 1\n\tv_min_i32_dpp %0, %1, %1 " CTRL " row_mask:0xf bank_mask:0xf" : "=v"(r) : "v"(v));          \
    return r;                                                                                                    \
  }
YKA_DPP_MIN(min_xor1, "quad_perm:[1,0,3,2]")            // with the neighbour in the pair
YKA_DPP_MIN(min_xor2, "quad_perm:[2,3,0,1]")            // with the other pair of the quad
YKA_DPP_MIN(min_oct, "row_half_mirror")                 // with the mirrored lane of 8: the other quad
YKA_DPP_MIN(min_ror4, "row_ror:4")                      // with the lane four further in the row of 16
YKA_DPP_MIN(min_ror8, "row_ror:8")
#undef YKA_DPP_MIN
// v + (w of the lane the control names), one instruction
#define YKA_DPP_ADD(NAME, CTRL)                                                                                  \
  __device__ __forceinline__ int NAME(int w, int v) {                                                            \
    int r;                                                                                                       \
    asm("s_nop 1\n\tv_add_u32_dpp %0, %1, %2 " CTRL " row_mask:0xf bank_mask:0xf" : "=v"(r) : "v"(w), "v"(v));  \
    return r;                                                                                                    \
  }
YKA_DPP_ADD(add_rot1, "quad_perm:[1,2,3,0]")            // w of the next lane of the quad (cyclic)
YKA_DPP_ADD(add_rot2, "quad_perm:[2,3,0,1]")
YKA_DPP_ADD(add_rot3, "quad_perm:[3,0,1,2]")
YKA_DPP_ADD(add_pos0, "quad_perm:[0,0,0,0]")            // w of lane 0 / 1 / 2 / 3 of the quad
YKA_DPP_ADD(add_pos1, "quad_perm:[1,1,1,1]")
YKA_DPP_ADD(add_pos2, "quad_perm:[2,2,2,2]")
YKA_DPP_ADD(add_pos3, "quad_perm:[3,3,3,3]")
#undef YKA_DPP_ADD

// Where the 256 states sit in a wave: 64 lanes x 4 slots, in one of two arrangements between which the costs alternate
// from step to step.  A state s is a member of group s & (U - 1) (U = 256 >> KK groups of 2^KK members: the states that
// can precede the same successors) and continues group s >> KK.  Write a lane as (r, q, i) = 16 r + 4 q + i.
//   5 bits, arrangement 0: lane = 8 (s >> 5) + (s & 7), slot = bits 3-4 of s.  A group's members are the lanes congruent
//     modulo 8; after the reduction (row rotation, row swap, half swap) all of them hold its minimum.  Arrangement 1:
//     lane = 8 (s & 7) + (s >> 5): exactly those lanes hold the states that continue that group, and a group's members
//     are now 8 adjacent lanes (three quad / half-mirror steps), which are the lanes of its successors in arrangement 0.
//   4 bits, arrangement 0: s = 16 (4 r + slot) + (lane & 15).  Members: lanes congruent modulo 16 (row swap, half swap); the minimum of
//     group 4 q + i then sits in lane (., q, i) of every row.  Arrangement 1: group (s & 15) = 4 r + i, continued group
//     (s >> 4) = 4 q + ((i + slot) & 3): a lane finds the four minima it needs in its own quad, rotated by the slot,
//     and a group's members are the four lanes (r, ., i) of a row (two row rotations).  Back in arrangement 0 the states
//     of lane (r, q, i), slot n continue group 4 r + n, whose minimum is in position n of the lane's own quad.
// No minimum is ever fetched through LDS.
template <int KK, int ARR>
__device__ __forceinline__ int state_at(int lane, int n) {
  const int r = lane >> 4, q = (lane >> 2) & 3, i = lane & 3;
  if constexpr (KK == 5) return ARR ? ((lane & 7) << 5) | (n << 3) | (lane >> 3) : ((lane >> 3) << 5) | (n << 3) | (lane & 7);
  else if constexpr (KK == 4) return ARR ? ((4 * q + ((i + n) & 3)) << 4) | (4 * r + i) : ((4 * r + n) << 4) | (lane & 15);
  else return (n << 6) | lane;
}
// the lane that holds the minimum of group g after the reduction in BOTH arrangements
template <int KK> __device__ __forceinline__ int keeper_lane(int g) { return KK == 5 ? 9 * g : 20 * (g >> 2) + (g & 3); }

// lane 0 walks the chosen path back from the best final state.  WORDS: word (t / 4) * 32 + u of bp holds, in byte t % 4,
// the predecessor index chosen at step t for the states that continue group u; otherwise byte t * 32 + u does.
template <int KK, bool WORDS>
__device__ __forceinline__ void walk_back(int best_state, const uint8_t* bp, uint8_t* st_out) {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  if ((threadIdx.x & 63) == 0) {
    int st = best_state;
    for (int t = 63; t >= 0; --t) {
      st_out[t] = (uint8_t)st;
      const int u = st >> KK;
      const int j = WORDS ? (int)((reinterpret_cast<const uint32_t*>(bp)[(t >> 2) * 32 + u] >> (8 * (t & 3))) & 255u) : (int)bp[t * 32 + u];
      st = (j << (8 - KK)) | u;
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
// The same walk for 4- and 5-bit fields, in parallel.  The step t -> t - 1 depends on the state only through the group
// u = state >> KK it continues (U = 256 >> KK values): state(t - 1) = (chosen[t][u] << (8 - KK)) | u.  The 64 steps are cut
// into 64 / U blocks of U steps; lane (block, u0) walks its block assuming it is entered in group u0 and keeps the
// states it passes.  A chain of 64 / U lane reads then finds, from the best final state downwards, the group in which
// every block really is entered, and the lanes that assumed right write their states.  bp in the word layout above.
template <int KK>
__device__ __forceinline__ void walk_back_blocks(int best_state, const uint8_t* bp, uint8_t* st_out) {
  constexpr int U = 256 >> KK, NB = 64 / U;            // steps per block, blocks
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  const int lane = threadIdx.x & 63, blk = lane / U, u0 = lane % U;
  const uint32_t* const words = reinterpret_cast<const uint32_t*>(bp) + (U / 4) * 32 * blk;
  int passed[U], u = u0;
#pragma unroll
  for (int i = 0; i < U; ++i) {                        // step t = U blk + U - 1 - i
    const int j = (int)((words[((U - 1 - i) >> 2) * 32 + u] >> (8 * ((U - 1 - i) & 3))) & 255u);
    passed[i] = (j << (8 - KK)) | u;                   // state(t - 1)
    u = passed[i] >> KK;
  }
  int entered = best_state >> KK, mine = 0;            // group in which the top block is entered
#pragma unroll
  for (int b = NB - 1; b >= 0; --b) {
    mine = blk == b ? entered : mine;
    entered = __builtin_amdgcn_readlane(u, __builtin_amdgcn_readfirstlane(U * b + entered));
  }
  if (lane == 0) st_out[63] = (uint8_t)best_state;
  if (u0 == mine) {
#pragma unroll
    for (int i = 0; i < U; ++i) {
      const int t1 = U * blk + U - 2 - i;              // t - 1
      if (t1 >= 0) st_out[t1] = (uint8_t)passed[i];
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
// smallest cost over the wave's 256 states, the smallest state among equal costs; sid[k] ascending in k
__device__ __forceinline__ int best_final(const int (&cost)[4], const int (&sid)[4]) {
  int bc = cost[0], bs = sid[0];
#pragma unroll
  for (int k = 1; k < 4; ++k) if (cost[k] < bc) { bc = cost[k]; bs = sid[k]; }
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int oc = __shfl_xor(bc, o, 64), os = __shfl_xor(bs, o, 64);
    if (oc < bc || (oc == bc && os < bs)) { bc = oc; bs = os; }
  }
  return bs;
}

// One chunk in one wave, 4- or 5-bit fields.  xi: the chunk's 64 integer targets (LDS), tab(s): table value of state s,
// bp: 64 x 32 bytes of LDS private to the wave, st_out: 64 bytes of LDS private to the wave.
// A state's cost is carried as key = cost * 2^KK + j with j the state's index among the members of its group, relative to
// a common offset (only differences decide): ONE minimum then yields the smallest cost and, among equal costs, the
// smallest predecessor.  At any step two states differ by at most two steps' worth of squared error, < 2 * 3148^2 (634 M
// in key units at 5 bits), and a step moves every key by -144 M ... +182 M, so the key fits 32 bits when the offset - the
// minimum of group 0 - is subtracted every fourth step.  States that cannot be reached yet start 40,000,000 above state
// 0: more than any path costs before every state is reachable (after two steps), like the reference's 2^30, and small
// enough for the key.
// a + x * b for |x|, |b| < 2^23, one full-rate instruction (x wave-uniform)
__device__ __forceinline__ int mad24(int x, int b, int a) {
  int r;
  asm("v_mad_i32_i24 %0, %1, %2, %3" : "=v"(r) : "s"(x), "v"(b), "v"(a));
  return r;
}
// (x - c)^2 = x^2 - 2 x c + c^2, and x^2 is common to all states of a step: a state's step cost in key units is
// a - x b with a = c^2 * 2^KK + j and b = 2 c * 2^KK, constants of the (lane, slot) in each arrangement
struct StepConsts { int a0[4], a1[4], b0[4], b1[4]; };
template <int KK, class Tab>
__device__ __forceinline__ StepConsts step_consts(Tab tab) {
  const int lane = threadIdx.x & 63;
  StepConsts C;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int s0 = state_at<KK, 0>(lane, k), s1 = state_at<KK, 1>(lane, k), c0 = tab(s0), c1 = tab(s1);
    C.a0[k] = ((c0 * c0) << KK) | (s0 >> (8 - KK)); C.b0[k] = (2 * c0) << KK;
    C.a1[k] = ((c1 * c1) << KK) | (s1 >> (8 - KK)); C.b1[k] = (2 * c1) << KK;
  }
  return C;
}
template <int KK>
__device__ __forceinline__ void wave_chunk(const int* xi, const StepConsts& C, uint8_t* bp, uint8_t* st_out) {
  static_assert(KK == 4 || KK == 5, "packed search: 4 or 5 bits");
  constexpr int U = 256 >> KK, kFar = 40000000, kLow = (1 << KK) - 1;
  const int lane = threadIdx.x & 63;
  const int xreg = xi[lane];                           // target t lives in lane t
  const int (&a0)[4] = C.a0, (&a1)[4] = C.a1, (&b0)[4] = C.b0, (&b1)[4] = C.b1;
  int sid[4], key[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    sid[k] = state_at<KK, 0>(lane, k);
    key[k] = ((sid[k] == 0 ? 0 : kFar) << KK) | (sid[k] >> (8 - KK));
  }
  // is this lane the keeper of a group, and of which: its record of chosen predecessors goes to LDS every four steps
  int kept = -1;
#pragma unroll
  for (int g = 0; g < U; ++g) kept = lane == keeper_lane<KK>(g) ? g : kept;
  uint32_t* const rec = reinterpret_cast<uint32_t*>(bp) + (kept < 0 ? 0 : kept);
#pragma unroll 1
  for (int t = 0; t < 64; t += 4) {
    uint32_t chosen4 = 0u;
#pragma unroll
    for (int h = 0; h < 4; h += 2) {
      {                                                // arrangement 0 -> 1
        int km = min(min(key[0], key[1]), min(key[2], key[3]));
        if constexpr (KK == 5) km = min_ror8(km);
        km = pair_min<32>(pair_min<16>(km));
        chosen4 = __builtin_amdgcn_alignbit((uint32_t)km, chosen4, 8);   // low byte of km enters at the top
        int m = km & ~kLow;                            // cost * 2^KK
        if (h == 0) m -= __builtin_amdgcn_readlane(m, 0);   // the common offset: group 0's minimum, once per four steps
        const int nx = -__builtin_amdgcn_readlane(xreg, t + h);
        if constexpr (KK == 5) {
#pragma unroll
          for (int k = 0; k < 4; ++k) key[k] = mad24(nx, b1[k], a1[k]) + m;
        } else {
          key[0] = mad24(nx, b1[0], a1[0]) + m;
          key[1] = add_rot1(m, mad24(nx, b1[1], a1[1]));
          key[2] = add_rot2(m, mad24(nx, b1[2], a1[2]));
          key[3] = add_rot3(m, mad24(nx, b1[3], a1[3]));
        }
      }
      {                                                // arrangement 1 -> 0
        int km = min(min(key[0], key[1]), min(key[2], key[3]));
        if constexpr (KK == 5) km = min_oct(min_xor2(min_xor1(km)));
        else km = min_ror8(min_ror4(km));
        chosen4 = __builtin_amdgcn_alignbit((uint32_t)km, chosen4, 8);
        const int m = km & ~kLow;
        const int nx = -__builtin_amdgcn_readlane(xreg, t + h + 1);
        if constexpr (KK == 5) {
#pragma unroll
          for (int k = 0; k < 4; ++k) key[k] = mad24(nx, b0[k], a0[k]) + m;
        } else {
          key[0] = add_pos0(m, mad24(nx, b0[0], a0[0]));
          key[1] = add_pos1(m, mad24(nx, b0[1], a0[1]));
          key[2] = add_pos2(m, mad24(nx, b0[2], a0[2]));
          key[3] = add_pos3(m, mad24(nx, b0[3], a0[3]));
        }
      }
    }
    if (kept >= 0) rec[(t >> 2) * 32] = chosen4 & (0x01010101u * (uint32_t)kLow);
  }
  int cost[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) cost[k] = key[k] >> KK;
  walk_back_blocks<KK>(best_final(cost, sid), bp, st_out);
}

// One chunk in one wave, 3-bit fields (32 groups of 8): unpacked costs, the group minima gathered across lanes.
__device__ __forceinline__ void wave_chunk3(const int* xi, const int (&ci4)[4], uint8_t* bp, uint8_t* st_out) {
  constexpr int KK = 3, U = 32, PER = 2;               // PER = predecessor indices j a lane step covers: j = l / U + PER * k
  const int lane = threadIdx.x & 63;
  const int xreg = xi[lane];
  int cost[4], sid[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) { sid[k] = lane + 64 * k; cost[k] = sid[k] == 0 ? 0 : 0x40000000; }
#pragma unroll 1
  for (int t = 0; t < 64; ++t) {
    const int mn = group_min<U>(min(min(cost[0], cost[1]), min(cost[2], cost[3])));
    int jb = 255;
#pragma unroll
    for (int k = 3; k >= 0; --k) jb = cost[k] == mn ? lane / U + PER * k : jb;
    jb = group_min<U>(jb);
    if (lane < U) bp[t * 32 + lane] = (uint8_t)jb;
    const int x = __builtin_amdgcn_readlane(xreg, t);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int m = __shfl(mn, (lane + 64 * k) >> KK, 64);   // lane u holds the minimum of group u
      const int dx = x - ci4[k];
      cost[k] = dx * dx + m;
    }
  }
  walk_back<KK, false>(best_final(cost, sid), bp, st_out);
}

// grid rows * nm, block 256: block = (row, multiplier); wave c = chunk c.  Writes the 256 states of the row under this
// multiplier and the 8 partial error sums to scratch.
__global__ void __launch_bounds__(256) tb_search_kernel(TbEncArgs A) {
  __shared__ float part8[8];
  __shared__ float rot_buf[256];
  __shared__ int target[256];
  __shared__ __align__(16) uint8_t back[4][64 * 32];
  __shared__ uint8_t chosen[256];
  __shared__ int16_t table[256];
  const int d = threadIdx.x, wave = d >> 6, lane = d & 63;
  const int row = blockIdx.x / A.nm, mult = blockIdx.x % A.nm;
  const Profile P{A.blob, A.desc, A.ngrp, A.mult_off};
  const RowRef R = locate_row(A, row, rot_buf);
  const GroupRec G = read_group(P, R.group);
  if (!G.present || R.pos < G.guard || G.mode != 0) return;                // uniform over the block: nothing to search
  // everything the search needs from memory is requested before the residual's block reductions
  const TableRec T = read_table(P, G);
  const auto tab = [&](int state) { return table_int(P, T, state); };
  StepConsts C{};
  int ci4[4] = {0, 0, 0, 0};
  if (G.bits == 5) C = step_consts<5>(tab);
  else if (G.bits == 4) C = step_consts<4>(tab);
  else {
#pragma unroll
    for (int k = 0; k < 4; ++k) ci4[k] = tab(lane + 64 * k);
  }
  const float mult_value = P.multiplier(mult);
  table[d] = (int16_t)tab(d);                            // published by the barriers of the block reductions
  const Residual Q = residual_of(part8, P, G, R.x);
  const float s = trial_scale(Q.rms, mult_value);
  // integer target of element d: the residual in units of s / 256, clamped
  target[d] = (int)fminf(fmaxf(rintf(__fmul_rn(__fdiv_rn(Q.r, s), 256.f)), -2048.f), 2048.f);
  __syncthreads();
  if (G.bits == 5) wave_chunk<5>(target + 64 * wave, C, back[wave], chosen + 64 * wave);
  else if (G.bits == 4) wave_chunk<4>(target + 64 * wave, C, back[wave], chosen + 64 * wave);
  else wave_chunk3(target + 64 * wave, ci4, back[wave], chosen + 64 * wave);
  // squared error of this multiplier: element d of the row is lane `lane` of wave `wave`; summed per run of 32 elements
  const int state = chosen[d];
  const float miss = __fsub_rn(Q.r, __fmul_rn(table_value((int)table[state], T.gain), s));
  float sq = __fmul_rn(miss, miss);
#pragma unroll
  for (int o = 16; o; o >>= 1) sq = __fadd_rn(sq, __shfl_xor(sq, o, 64));
  const size_t job = (size_t)row * A.nm + mult;
  if ((d & 31) == 0) reinterpret_cast<float*>(A.scr + A.scr_w_ofs)[job * 8 + (d >> 5)] = sq;
  A.scr[job * 256 + d] = (uint8_t)state;
}

// word d of a row's MSB-first stream of KB-bit fields: the fields that overlap bits [32 d, 32 d + 32)
template <int KB>
__device__ __forceinline__ uint32_t pack_word(const uint8_t* fld, int d) {
  const int e0 = (32 * d) / KB;                          // first field with bits in the word (division by a constant)
  uint32_t w = 0u;
#pragma unroll
  for (int k = 0; k < 32 / KB + 2; ++k) {
    const int e = e0 + k, sh = 32 * d + 32 - KB * (e + 1);   // distance of the field's last bit from the word's last bit
    if (e < 256 && sh > -KB) w |= sh >= 0 ? (uint32_t)fld[e] << sh : (uint32_t)fld[e] >> -sh;
  }
  return w;
}

// what a row is stored as: one field per element, the field width, the row scale
struct Coded { int field, bits; float scale, value; bool any; };
// flat groups: symmetric int4 with scale max|r| / 7 (src/kvq_fast.cuh:194-198)
__device__ __forceinline__ Coded code_flat(float* part8, float r) {
  const float top = block_fold<MaxOp>(part8, fabsf(r), 0.f);
  float step = __fdiv_rn(top, 7.f);
  if (step == 0.f) step = 1.f;
  const float q = fminf(fmaxf(rintf(__fdiv_rn(r, step)), -7.f), 7.f);
  return Coded{(int)q + 8, 4, step, __fmul_rn(q, step), true};
}
// trellis groups: the multiplier whose search left the smallest squared error (its 8 partial sums added in order from 0;
// the first of equal errors), the state the search chose for this element under it.  What that needs from memory is
// requested before the residual is computed, for all multipliers at once (the choice then costs no further round trip):
// the states of this element, and - by thread i < multipliers - multiplier i and the error total of its search.
constexpr int kMaxMult = 16;
struct SearchResults { int state[kMaxMult]; };
__device__ __forceinline__ SearchResults fetch_search_results(const TbEncArgs& A, const Profile& P, int row, float* totals, float* mults) {
  SearchResults S;
  const int d = threadIdx.x;
#pragma unroll
  for (int i = 0; i < kMaxMult; ++i) S.state[i] = i < A.nm ? (int)A.scr[((size_t)row * A.nm + i) * 256 + d] : 0;
  if (d < A.nm) {
    const float* err = reinterpret_cast<const float*>(A.scr + A.scr_w_ofs) + ((size_t)row * A.nm + d) * 8;
    float total = 0.f;
#pragma unroll
    for (int k = 0; k < 8; ++k) total = __fadd_rn(total, err[k]);
    totals[d] = total;
    mults[d] = P.multiplier(d);
  }
  return S;                                              // totals / mults: visible after the next barrier
}
__device__ __forceinline__ Coded code_trellis(const TbEncArgs& A, const Profile& P, const GroupRec& G, const Residual& Q, const SearchResults& S,
                                              const float* totals, const float* mults) {
  int keep = 0; float least = totals[0];
  for (int i = 1; i < A.nm; ++i) { const float total = totals[i]; if (total < least) { least = total; keep = i; } }
  const float s = trial_scale(Q.rms, mults[keep]);
  int state = 0;
#pragma unroll
  for (int i = 0; i < kMaxMult; ++i) state = i == keep ? S.state[i] : state;
  float value = 0.f;
  if (A.yout) { const TableRec T = read_table(P, G); value = __fmul_rn(table_value(table_int(P, T, state), T.gain), s); }
  return Coded{state & ((1 << G.bits) - 1), G.bits, s, value, true};
}

// grid rows, block 256: codes the row (best multiplier of the search, or the flat quantizer), rebuilds what it decodes to,
// packs the fields, stores payload / scale / projection coefficients
__global__ void __launch_bounds__(256) tb_select_kernel(TbEncArgs A) {
  __shared__ float part8[8];
  __shared__ float rot_buf[256];
  __shared__ uint8_t fld[256];
  __shared__ float totals[kMaxMult], mults[kMaxMult];
  const int d = threadIdx.x, row = blockIdx.x;
  const Profile P{A.blob, A.desc, A.ngrp, A.mult_off};
  const RowRef R = locate_row(A, row, rot_buf);
  const GroupRec G = read_group(P, R.group);
  Coded C{0, 4, 1.f, R.x, false};
  float rebuilt = R.x;                                   // rows that stay uncoded come back as they are
  unsigned coef_bits = 0u;
  if (G.present && R.pos >= G.guard) {
    SearchResults S{};
    if (G.mode == 0) S = fetch_search_results(A, P, row, totals, mults);
    const Residual Q = residual_of(part8, P, G, R.x);   // its barriers publish totals / mults
    if (G.mode == 1) C = code_flat(part8, Q.r);
    else if (G.mode == 0) C = code_trellis(A, P, G, Q, S, totals, mults);
    else C.value = Q.r;
    rebuilt = C.value;
#pragma unroll
    for (int k = 0; k < 2; ++k) if (k < G.ndir) rebuilt = __fadd_rn(rebuilt, __fmul_rn(Q.coef[k], Q.dir[k]));
    if (G.has_mean) rebuilt = __fadd_rn(rebuilt, Q.mean);
    coef_bits = (unsigned)__half_as_ushort(__float2half_rn(Q.coef[0])) | ((unsigned)__half_as_ushort(__float2half_rn(Q.coef[1])) << 16);
  }
  const bool storable = A.yin || (R.valid && R.pos >= 0 && R.pos < A.max_ctx && (A.pos_limit == 0 || R.pos < A.pos_limit));
  uint8_t* const plane = R.is_v ? A.pay1 : A.pay0;
  if (plane && storable) {
    uint32_t* const words = reinterpret_cast<uint32_t*>(plane + R.container + R.index * (size_t)A.stride);
    fld[d] = (uint8_t)C.field;
    __syncthreads();
    if (d < (A.stride >> 2)) {
      uint32_t w = 0u;
      if (C.any && d < 8 * C.bits) w = C.bits == 5 ? pack_word<5>(fld, d) : C.bits == 4 ? pack_word<4>(fld, d) : pack_word<3>(fld, d);
      words[d] = w;
    }
    if (d == 0) {
      float* const scales = R.is_v ? A.scl1 : A.scl0;
      if (scales) reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(scales) + R.container)[R.index] = C.scale;
      if (A.side) { A.side[2 * R.index] = __float_as_uint(C.scale); A.side[2 * R.index + 1] = coef_bits; }
      if (A.coded) A.coded[R.index] = C.any ? 1 : 0;
    }
  }
  if (A.yout) A.yout[R.index * 256 + d] = rebuilt;
}

// n <= 13 bits that start at bit `first` of an MSB-first stream of words (bits past the last word read as zero)
__device__ __forceinline__ unsigned stream_field(const uint32_t* words, int nwords, int first, int n) {
  const int w = first >> 5, used = first & 31;
  const uint32_t hi = words[w], lo = w + 1 < nwords ? words[w + 1] : 0u;
  const uint32_t window = used ? (hi << used) | (lo >> (32 - used)) : hi;   // the 32 bits that start at `first`
  return window >> (32 - n);
}
// decoder (src/kvq_attn.cuh:46-75): grid rows, block 256.  The state of element d is the last 8 bits of the stream up to
// the end of its field, cut at the start of its chunk of 64 elements.
__global__ void __launch_bounds__(256) tb_unpack_kernel(const uint8_t* blob, const int* grp, const int* pos, const uint8_t* pay, const uint32_t* side,
                                                        int stride, const float* yin, float* y) {
  __shared__ float values[256];
  const int row = blockIdx.x, d = threadIdx.x;
  const Profile P{blob};
  const GroupRec G = read_group(P, grp[row]);
  float out = yin ? yin[(size_t)row * 256 + d] : 0.f;
  if (G.present && pos[row] >= G.guard && G.mode <= 1) {                    // uniform over the block
    const uint32_t* words = reinterpret_cast<const uint32_t*>(pay + (size_t)row * stride);
    const float s = __uint_as_float(side[2 * (size_t)row]);
    const unsigned coef_bits = side[2 * (size_t)row + 1];
    float v;
    if (G.mode == 1) {
      v = __fmul_rn((float)((int)stream_field(words, 32, 4 * d, 4) - 8), s);
    } else {
      const TableRec T = read_table(P, G);
      values[d] = table_value(table_int(P, T, d), T.gain);
      __syncthreads();
      const int end = G.bits * (d + 1), chunk_start = G.bits * (d & ~63), begin = max(end - 8, chunk_start);
      v = __fmul_rn(values[stream_field(words, 8 * G.bits, begin, end - begin)], s);
    }
    const float coef[2] = {__half2float(__ushort_as_half((unsigned short)(coef_bits & 0xffffu))), __half2float(__ushort_as_half((unsigned short)(coef_bits >> 16)))};
#pragma unroll
    for (int k = 0; k < 2; ++k) if (k < G.ndir) v = __fadd_rn(v, __fmul_rn(coef[k], P.f16_at(G.dir_off + 512u * (unsigned)k + 2u * (unsigned)d)));
    if (G.has_mean) v = __fadd_rn(v, P.f16_at(G.mean_off + 2u * (unsigned)d));
    out = v;
  }
  y[(size_t)row * 256 + d] = out;
}

}  // namespace

void launch_tb_encode(const TbEncArgs& A, hipStream_t st) {
  if (A.nrow <= 0) return;
  if (A.has_trellis) hipLaunchKernelGGL(tb_search_kernel, dim3(A.nrow * A.nm), dim3(256), 0, st, A);
  hipLaunchKernelGGL(tb_select_kernel, dim3(A.nrow), dim3(256), 0, st, A);
}
void launch_tb_unpack(const uint8_t* blob, const int* grp, const int* pos, const uint8_t* pay, const uint32_t* side, int stride, const float* yin,
                      float* y, int rows, hipStream_t st) {
  if (rows > 0) hipLaunchKernelGGL(tb_unpack_kernel, dim3(rows), dim3(256), 0, st, blob, grp, pos, pay, side, stride, yin, y);
}

}  // namespace yka
