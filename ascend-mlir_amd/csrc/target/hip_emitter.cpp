#include "hip_emitter.h"

#include <cstddef>
#include <cstdio>
#include <cstring>
#include <sstream>
#include <vector>

namespace afir_target {

using namespace afir_region;

namespace {

// Device helpers of every emitted file.  Builtins only: the file compiles with
// -nogpuinc.
const char *const kPrelude = R"HIP(
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
#define DEV static __attribute__((device)) inline __attribute__((always_inline))
#define KERNEL extern "C" __attribute__((global)) __attribute__((amdgpu_flat_work_group_size(256, 256)))
// eight workgroups of 256 lanes per compute unit: at most 64 vector registers
#define PHASED_KERNEL KERNEL __attribute__((amdgpu_waves_per_eu(8, 8)))

struct SpecInput {
  const void *base;
  const void *index;
  long long stride[3];
  long long offset;
  long long gstride;
  long long gextent;
  int vec;
  int gvec;
};
struct SpecArgs {
  long long size[3];
  void *out;
  int *error_flag;
  int out_vec;
  int lanes_log2;
  int grid;
  int column_blocks;
  SpecInput in[8];
  float extent_const[8];
  int hold_ticks;
  int first_block;
};

DEV float as_f32(unsigned u) { return __builtin_bit_cast(float, u); }
DEV unsigned as_u32(float f) { return __builtin_bit_cast(unsigned, f); }
DEV float fmax_ieee(float a, float b) { return __builtin_elementwise_maximum(a, b); }
DEV float fmin_ieee(float a, float b) { return __builtin_elementwise_minimum(a, b); }

// A float32 value as the compiler may not look into it.  Without this, the conversion of a
// product to f16 is selected as one v_fma_mixlo_f16 with a zero addend: a single rounding of the
// exact product where the program asks for two (to float32, then to f16), and +0 where the
// product is -0.
DEV float f32_value(float x) {
  asm("" : "+v"(x));
  return x;
}
// ---- element access: float32 in registers, one round-to-nearest-even on store
DEV float ld_f32(const void *b, long long i) { return ((const float *)b)[i]; }
DEV float ld_f16(const void *b, long long i) {
  return (float)__builtin_bit_cast(_Float16, ((const unsigned short *)b)[i]);
}
DEV float ld_bf16(const void *b, long long i) { return as_f32((unsigned)((const unsigned short *)b)[i] << 16); }
DEV long long ld_i32(const void *b, long long i) { return ((const int *)b)[i]; }
DEV long long ld_i64(const void *b, long long i) { return ((const long long *)b)[i]; }
DEV unsigned bf16_rne(float f) {
  const unsigned u = as_u32(f);
  const unsigned r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
  return (f != f) ? ((u >> 16) | 0x40u) : r;
}
// round to the narrower type (nearest even) and widen again
DEV float rt_f16(float x) { return (float)(_Float16)f32_value(x); }
DEV float rt_bf16(float x) { return as_f32(bf16_rne(x) << 16); }
DEV float rt_f32(float x) { return x; }
DEV void st_f32(void *o, long long i, float x) { ((float *)o)[i] = x; }
DEV void st_f16(void *o, long long i, float x) {
  ((unsigned short *)o)[i] = __builtin_bit_cast(unsigned short, (_Float16)f32_value(x));
}
DEV void st_bf16(void *o, long long i, float x) { ((unsigned short *)o)[i] = (unsigned short)bf16_rne(x); }

// ---- 128-bit access; NT: the tensor is read exactly once by the launch
template <bool NT> DEV f32x4 ld128(const f32x4 *p) { return NT ? __builtin_nontemporal_load(p) : *p; }
template <bool NT> DEV u32x4 ld128(const u32x4 *p) { return NT ? __builtin_nontemporal_load(p) : *p; }
template <int V, bool NT> DEV void ldv_f32(const void *b, long long i, float (&v)[V]) {
  const f32x4 *p = (const f32x4 *)((const float *)b + i);
#pragma unroll
  for (int q = 0; q < V / 4; ++q) {
    const f32x4 a = ld128<NT>(p + q);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[4 * q + e] = a[e];
  }
}
template <int V, bool NT> DEV void ldv_f16(const void *b, long long i, float (&v)[V]) {
  const u32x4 *p = (const u32x4 *)((const unsigned short *)b + i);
#pragma unroll
  for (int q = 0; q < V / 8; ++q) {
    const u32x4 raw = ld128<NT>(p + q);
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const unsigned word = raw[d];   // a copy: bit_cast of a vector element reads element 0
      const f16x2 h = __builtin_bit_cast(f16x2, word);
      v[8 * q + 2 * d] = (float)h.x;
      v[8 * q + 2 * d + 1] = (float)h.y;
    }
  }
}
template <int V, bool NT> DEV void ldv_bf16(const void *b, long long i, float (&v)[V]) {
  const u32x4 *p = (const u32x4 *)((const unsigned short *)b + i);
#pragma unroll
  for (int q = 0; q < V / 8; ++q) {
    const u32x4 raw = ld128<NT>(p + q);
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      v[8 * q + 2 * d] = as_f32(raw[d] << 16);
      v[8 * q + 2 * d + 1] = as_f32(raw[d] & 0xffff0000u);
    }
  }
}
template <int V> DEV void stv_f32(void *o, long long i, const float (&v)[V]) {
  f32x4 *p = (f32x4 *)((float *)o + i);
#pragma unroll
  for (int q = 0; q < V / 4; ++q) {
    f32x4 a;
#pragma unroll
    for (int e = 0; e < 4; ++e) a[e] = v[4 * q + e];
    __builtin_nontemporal_store(a, p + q);
  }
}
template <int V> DEV void stv_f16(void *o, long long i, const float (&v)[V]) {
  u32x4 *p = (u32x4 *)((unsigned short *)o + i);
#pragma unroll
  for (int q = 0; q < V / 8; ++q) {
    u32x4 w;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      f16x2 h;
      h.x = (_Float16)f32_value(v[8 * q + 2 * d]);
      h.y = (_Float16)f32_value(v[8 * q + 2 * d + 1]);
      w[d] = __builtin_bit_cast(unsigned, h);
    }
    __builtin_nontemporal_store(w, p + q);
  }
}
template <int V> DEV void stv_bf16(void *o, long long i, const float (&v)[V]) {
  u32x4 *p = (u32x4 *)((unsigned short *)o + i);
#pragma unroll
  for (int q = 0; q < V / 8; ++q) {
    u32x4 w;
#pragma unroll
    for (int d = 0; d < 4; ++d)
      w[d] = (bf16_rne(v[8 * q + 2 * d]) & 0xffffu) | (bf16_rne(v[8 * q + 2 * d + 1]) << 16);
    __builtin_nontemporal_store(w, p + q);
  }
}

// ---- integer regions: 32-bit two's complement values, i16 sign-extended on
// load and truncated on store
DEV int ldd_i32(const void *b, long long i) { return ((const int *)b)[i]; }
DEV int ldd_i16(const void *b, long long i) { return (int)((const short *)b)[i]; }
DEV void st_i32(void *o, long long i, int x) { ((int *)o)[i] = x; }
DEV void st_i16(void *o, long long i, int x) { ((short *)o)[i] = (short)x; }
template <int V, bool NT> DEV void ldv_i32(const void *b, long long i, int (&v)[V]) {
  const u32x4 *p = (const u32x4 *)((const int *)b + i);
#pragma unroll
  for (int q = 0; q < V / 4; ++q) {
    const u32x4 raw = ld128<NT>(p + q);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[4 * q + e] = (int)raw[e];
  }
}
template <int V, bool NT> DEV void ldv_i16(const void *b, long long i, int (&v)[V]) {
  const u32x4 *p = (const u32x4 *)((const short *)b + i);
#pragma unroll
  for (int q = 0; q < V / 8; ++q) {
    const u32x4 raw = ld128<NT>(p + q);
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const unsigned word = raw[d];
      v[8 * q + 2 * d] = (int)(word << 16) >> 16;
      v[8 * q + 2 * d + 1] = (int)word >> 16;
    }
  }
}
template <int V> DEV void stv_i32(void *o, long long i, const int (&v)[V]) {
  u32x4 *p = (u32x4 *)((int *)o + i);
#pragma unroll
  for (int q = 0; q < V / 4; ++q) {
    u32x4 a;
#pragma unroll
    for (int e = 0; e < 4; ++e) a[e] = (unsigned)v[4 * q + e];
    __builtin_nontemporal_store(a, p + q);
  }
}
template <int V> DEV void stv_i16(void *o, long long i, const int (&v)[V]) {
  u32x4 *p = (u32x4 *)((short *)o + i);
#pragma unroll
  for (int q = 0; q < V / 8; ++q) {
    u32x4 w;
#pragma unroll
    for (int d = 0; d < 4; ++d)
      w[d] = ((unsigned)v[8 * q + 2 * d] & 0xffffu) | ((unsigned)v[8 * q + 2 * d + 1] << 16);
    __builtin_nontemporal_store(w, p + q);
  }
}

// ---- one 16-byte chunk <-> W values (the phased kernels keep packed results in registers)
DEV void cvt_f32(const u32x4 raw, float (&v)[4]) {
#pragma unroll
  for (int e = 0; e < 4; ++e) v[e] = as_f32(raw[e]);
}
DEV void cvt_f16(const u32x4 raw, float (&v)[8]) {
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const unsigned word = raw[d];
    const f16x2 h = __builtin_bit_cast(f16x2, word);
    v[2 * d] = (float)h.x;
    v[2 * d + 1] = (float)h.y;
  }
}
DEV void cvt_bf16(const u32x4 raw, float (&v)[8]) {
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    v[2 * d] = as_f32(raw[d] << 16);
    v[2 * d + 1] = as_f32(raw[d] & 0xffff0000u);
  }
}
DEV void cvt_i32(const u32x4 raw, int (&v)[4]) {
#pragma unroll
  for (int e = 0; e < 4; ++e) v[e] = (int)raw[e];
}
DEV void cvt_i16(const u32x4 raw, int (&v)[8]) {
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const unsigned word = raw[d];
    v[2 * d] = (int)(word << 16) >> 16;
    v[2 * d + 1] = (int)word >> 16;
  }
}
DEV u32x4 pk_f32(const float (&v)[4]) {
  u32x4 w;
#pragma unroll
  for (int e = 0; e < 4; ++e) w[e] = as_u32(v[e]);
  return w;
}
DEV u32x4 pk_f16(const float (&v)[8]) {
  u32x4 w;
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    f16x2 h;
    h.x = (_Float16)f32_value(v[2 * d]);
    h.y = (_Float16)f32_value(v[2 * d + 1]);
    w[d] = __builtin_bit_cast(unsigned, h);
  }
  return w;
}
DEV u32x4 pk_bf16(const float (&v)[8]) {
  u32x4 w;
#pragma unroll
  for (int d = 0; d < 4; ++d) w[d] = (bf16_rne(v[2 * d]) & 0xffffu) | (bf16_rne(v[2 * d + 1]) << 16);
  return w;
}
DEV u32x4 pk_i32(const int (&v)[4]) {
  u32x4 w;
#pragma unroll
  for (int e = 0; e < 4; ++e) w[e] = (unsigned)v[e];
  return w;
}
DEV u32x4 pk_i16(const int (&v)[8]) {
  u32x4 w;
#pragma unroll
  for (int d = 0; d < 4; ++d) w[d] = ((unsigned)v[2 * d] & 0xffffu) | ((unsigned)v[2 * d + 1] << 16);
  return w;
}

// ---- sum over the 64 lanes of a wavefront, fixed order: quad butterflies,
// half-row and row mirrors, then the four row totals
template <int C> DEV float dpp_add(float v) {
  const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), C, 0xf, 0xf, true);
  return v + __builtin_bit_cast(float, moved);
}
DEV float wave_sum(float v) {
  v = dpp_add<0xB1>(v);
  v = dpp_add<0x4E>(v);
  v = dpp_add<0x141>(v);
  v = dpp_add<0x140>(v);
  const int iv = __builtin_bit_cast(int, v);
  const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 0));
  const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 16));
  const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 32));
  const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 48));
  return (r0 + r1) + (r2 + r3);
}
// ---- a source row staged in LDS (dynamic: the launch gives its size), read back by index
extern __attribute__((shared)) __attribute__((aligned(16))) unsigned short afir_stage[];
typedef __attribute__((address_space(3))) const float lds_f32;
typedef __attribute__((address_space(3))) const int lds_i32;
typedef __attribute__((address_space(3))) const short lds_i16;
DEV float stage_f16(long long i) { return (float)__builtin_bit_cast(_Float16, afir_stage[i]); }
DEV float stage_bf16(long long i) { return as_f32((unsigned)afir_stage[i] << 16); }
DEV float stage_f32(long long i) { return ((lds_f32 *)afir_stage)[i]; }
DEV int staged_i16(long long i) { return (int)((lds_i16 *)afir_stage)[i]; }
DEV int staged_i32(long long i) { return ((lds_i32 *)afir_stage)[i]; }

// ---- sum over aligned sets of `lanes` (a power of two below 64) lanes: butterfly, fixed order.
// The lanes of a set are all active or all inactive.
DEV float lanes_sum(float v, int lane, int lanes) {
  for (int m = lanes >> 1; m >= 1; m >>= 1)
    v += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ m) << 2, __builtin_bit_cast(int, v)));
  return v;
}
)HIP";

const char *typeTag(ElemType t) {
  switch (t) {
    case ElemType::F16: return "f16";
    case ElemType::BF16: return "bf16";
    case ElemType::F32: return "f32";
    case ElemType::I32: return "i32";
    case ElemType::I64: return "i64";
    case ElemType::I16: return "i16";
  }
  return "f32";
}

std::string floatLiteral(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  char buf[64];
  std::snprintf(buf, sizeof buf, "as_f32(0x%08xu) /* %g */", u, (double)f);
  return buf;
}

// A constant of an integer region (validated to be a 32-bit integer).
std::string intLiteral(float f) {
  const long long v = (long long)f;
  return v == -2147483648ll ? std::string("(-2147483647 - 1)") : "(" + std::to_string(v) + ")";
}

// One distinct operand read of a segment.
struct Operand {
  int slot = 0;            // index into SpecArgs::in (the first push that reads it)
  ElemType type = ElemType::F32;
  enum Step { Broadcast, Contiguous, Strided } step = Broadcast;
  int gatherDim = -1;      // iteration dim that indexes the index tensor
  ElemType gatherType = ElemType::I64;
  bool usesDim[kMaxRank] = {false, false, false};
  bool readOnce = false;   // every iteration dim addresses it: no reuse across the launch
  // Strided along the innermost iteration dim but contiguous along another one
  // (a transposed read): staged through an LDS tile when the segment is tiled.
  int contiguousDim = -1;  // the iteration dim the operand's innermost dim follows, else -1
  bool tiled = false;
  int tileSlot = 0;        // which LDS tile
  // the operand in the kernel that separates reads from writes (specPhased)
  enum Phase { PhaseScalar, PhaseStreamed, PhaseVector, PhaseOther } phase = PhaseOther;
  int vectorSlot = 0;      // PhaseVector: which stretch of the LDS
};

bool sameRead(const Op &a, const Op &b) {
  if (a.arg != b.arg || a.map.size() != b.map.size() || a.slice.size() != b.slice.size()) return false;
  for (size_t i = 0; i < a.map.size(); ++i) {
    const MapResult &x = a.map[i], &y = b.map[i];
    if (x.kind != y.kind || x.iterDim != y.iterDim || x.constant != y.constant || x.indexArg != y.indexArg)
      return false;
  }
  for (size_t i = 0; i < a.slice.size(); ++i)
    if (a.slice[i].arg != b.slice[i].arg || a.slice[i].dim != b.slice[i].dim ||
        a.slice[i].constant != b.slice[i].constant)
      return false;
  return true;
}

constexpr int kMaxTiles = 2;

struct Value {
  std::string name;
  bool scalar = false;
  std::string at() const { return scalar ? name : name + "[u][e]"; }
};

// A lane's share of one pass over a row: U groups of W consecutive elements,
// the groups 2^lanes_log2 * W elements apart, so that every load or store
// instruction of a wavefront covers one contiguous run of memory.
class SegmentEmitter {
 public:
  SegmentEmitter(const Program &p, int index, std::ostringstream &os, const EmitOptions &options = EmitOptions())
      : p_(p), seg_(p.segments[index]), index_(index), os_(os), opt_(options) {}

  std::string run() {
    if (!seg_.ops.empty() && seg_.ops[0].code == OpCode::Matmul)
      return "matmul segments run on the hand-written MFMA kernels";
    const SpecShape shape = specShape(p_, index_, opt_);
    W_ = shape.width;
    U_ = shape.unroll;
    analyze();
    if ((int)pushSlot_.size() > kSpecMaxInputs) return "more than 8 operand reads in a segment";
    if (tiled()) {
      U_ = opt_.tileQ / 8 / W_;   // eight lanes cover a tile row
      emitBodyTiled();
    } else {
      emitBody();
      if (reduce_) {
        emitBodyRowGroup();
        emitBodyLongRows();
        emitBodySplitRows();
      }
      if (phased_.eligible) emitBodyPhased();
      if (U_ > 1) {
        // the same with one group per lane, for short rows
        const int wide = U_;
        U_ = 1;
        slim_ = true;
        emitBody();
        slim_ = false;
        U_ = wide;
        hasSlim_ = true;
      }
      if (stageOperand_ >= 0) {
        stage_ = true;
        emitBody();
        stageWave_ = true;    // the same with a wavefront per row, for short rows
        emitBody();
        stageWave_ = false;
        stage_ = false;
      }
      {
        // the same with one element per group, for tensors whose rows do not start on 16-byte
        // boundaries: consecutive lanes take consecutive elements, so every load and store
        // instruction of a wavefront still covers one contiguous run
        const int wideU = U_, wideW = W_;
        U_ = kSpecElementUnroll;
        W_ = 1;
        elem_ = true;
        emitBody();
        elem_ = false;
        U_ = wideU;
        W_ = wideW;
      }
    }
    emitWrappers();
    return "";
  }

 private:
  void collectOperands() {
    int slot = 0;
    std::vector<const Op *> firsts;
    for (const Op &op : seg_.ops) {
      if (op.code != OpCode::Push) continue;
      int found = -1;
      for (size_t i = 0; i < firsts.size(); ++i)
        if (sameRead(*firsts[i], op)) found = (int)i;
      if (found < 0) {
        Operand o;
        o.slot = slot;
        o.type = p_.args[op.arg].type;
        int lastHits = 0;
        bool lastInnermost = false;
        for (size_t d = 0; d < op.map.size(); ++d) {
          const MapResult &m = op.map[d];
          if (m.kind == MapResult::IterDim) {
            o.usesDim[m.iterDim] = true;
            if (m.iterDim == last_) {
              ++lastHits;
              lastInnermost = d + 1 == op.map.size();
            }
          } else if (m.kind == MapResult::Gather) {
            o.gatherDim = m.iterDim;
            o.gatherType = p_.args[m.indexArg].type;
          }
        }
        o.step = lastHits == 0 ? Operand::Broadcast
                               : (lastHits == 1 && lastInnermost ? Operand::Contiguous : Operand::Strided);
        if (o.step == Operand::Strided && lastHits == 1 && o.gatherDim < 0 && !op.map.empty() &&
            op.map.back().kind == MapResult::IterDim && op.map.back().iterDim != last_) {
          int hits = 0;
          for (const MapResult &m : op.map)
            if (m.kind == MapResult::IterDim && m.iterDim == op.map.back().iterDim) ++hits;
          if (hits == 1) o.contiguousDim = op.map.back().iterDim;
        }
        o.readOnce = true;
        for (int k = 0; k < rank_; ++k)
          if (!o.usesDim[k] && o.gatherDim != k) o.readOnce = false;
        if (o.gatherDim >= 0) o.readOnce = false;   // gathered rows may repeat
        found = (int)firsts.size();
        firsts.push_back(&op);
        operands_.push_back(o);
      }
      pushSlot_.push_back(found);
      ++slot;
    }
    // a parallel segment with transposed reads is walked in tiles of
    // kTileP x kTileQ over (that dim, innermost dim); up to two such operands
    // go through LDS, all along the same dim
    tileDim_ = -1;
    int tiles = 0;
    if (!reduce_)
      for (Operand &o : operands_)
        if (o.contiguousDim >= 0 && (tileDim_ < 0 || tileDim_ == o.contiguousDim) && tiles < kMaxTiles) {
          tileDim_ = o.contiguousDim;
          o.tiled = true;
          o.tileSlot = tiles++;
        }
    numTiles_ = tiles;
    // Non-temporal loads pay when reads dominate the traffic (two full-size inputs per output:
    // 6.25 against 5.8 TB/s; a row sum 3 %).  A segment that writes about as many bytes as it
    // streams in (one full-size input per output) keeps ordinary loads next to its non-temporal
    // stores: from HBM the two measure within 2 % of each other, and inputs that a previous launch
    // left in the 256 MB last-level cache are found there only by ordinary loads (a copy cycling
    // over 256 MiB: 6.7 against 6.0 TB/s, the tiled transpose 6.5 against 5.5).
    if (!reduce_) {
      size_t streamed = 0;
      for (const Operand &o : operands_)
        if (o.readOnce) streamed += elemTypeBytes(o.type);
      if (streamed * 4 <= elemTypeBytes(p_.output().type) * 5)
        for (Operand &o : operands_) o.readOnce = false;
    }
    // a gather along the innermost dim from rows of a matrix (the index tensor picks the column):
    // the source row can be staged in LDS and gathered from there
    stageOperand_ = -1;
    if (!reduce_ && rank_ == 2 && tileDim_ < 0) {
      int found = -1, count = 0;
      for (size_t i = 0; i < operands_.size(); ++i)
        if (operands_[i].gatherDim == last_) {
          ++count;
          found = (int)i;
        }
      if (count == 1 && operands_[found].usesDim[0] && operands_[found].step == Operand::Broadcast) stageOperand_ = found;
    }
    classifyForPhases();
  }

  // Whether the segment has the form that separates its reads from its writes (specPhased), and
  // what each operand is in it.
  void classifyForPhases() {
    phased_ = SpecPhased();
    if (reduce_ || tileDim_ >= 0 || stageOperand_ >= 0) return;
    const size_t es = elemTypeBytes(p_.output().type);
    int streamed = 0, vectors = 0;
    for (Operand &o : operands_) {
      o.phase = Operand::PhaseOther;
      if (o.gatherDim == last_) return;
      if (o.step == Operand::Broadcast) {
        o.phase = Operand::PhaseScalar;
        continue;
      }
      if (o.step != Operand::Contiguous || elemTypeBytes(o.type) != es) return;
      bool all = true, none = o.gatherDim < 0;
      for (int k = 0; k < last_; ++k) {
        if (!(o.usesDim[k] || o.gatherDim == k)) all = false;
        if (o.usesDim[k]) none = false;
      }
      if (all) {
        o.phase = Operand::PhaseStreamed;
        ++streamed;
      } else if (none) {
        o.phase = Operand::PhaseVector;
        o.vectorSlot = vectors++;
      } else {
        return;
      }
    }
    if (streamed < 1 || streamed > 2 || vectors > kSpecPhasedMaxVectors) return;
    phased_.eligible = true;
    phased_.streamed = streamed;
    phased_.vectors = vectors;
    phased_.elemBytes = (int)es;
  }

 public:
  bool tiled() const { return tileDim_ >= 0; }
  SpecPhased phased() const { return phased_; }
  // SpecArgs::in slot of the operand whose source rows the staged kernels keep in LDS, else -1
  int stagedSlot() const { return stageOperand_ < 0 ? -1 : operands_[stageOperand_].slot; }
  ElemType stagedType() const { return stageOperand_ < 0 ? ElemType::F32 : operands_[stageOperand_].type; }
  int tileDim() const { return tileDim_; }
  unsigned tiledInputs() const {
    unsigned mask = 0;
    for (const Operand &o : operands_)
      if (o.tiled) mask |= 1u << o.slot;
    return mask;
  }
  void analyze() {
    integer_ = isRegionInt(p_.output().type);
    narrow_ = p_.output().type == ElemType::I16;
    rank_ = seg_.rank;
    last_ = rank_ - 1;
    reduce_ = seg_.reduces();
    collectOperands();
  }

 private:
  std::string in(const Operand &o) const { return "R.in[" + std::to_string(o.slot) + "]"; }
  std::string id(const Operand &o) const { return std::to_string(o.slot); }
  void line(int depth, const std::string &text) { os_ << std::string(2 * depth, ' ') << text << "\n"; }
  void unroll() { os_ << "#pragma unroll\n"; }

  // Row-invariant part of every operand: its position without the innermost
  // dim, the index of a gather along an outer dim, the value of an operand that
  // is broadcast along the innermost dim.
  // hoisted_: the variables were declared by emitOperandDeclarations and are assigned here.
  void emitRowInvariants(int d) {
    const std::string cll = hoisted_ ? "" : "const long long ", cb = hoisted_ ? "" : "const bool ",
                      cv = hoisted_ ? "" : "const " + ct() + " ";
    for (const Operand &o : operands_) {
      if (keepRowConstants_ && rowConstant(o)) continue;
      const std::string u = id(o), r = in(o);
      std::string pos = "(I)" + r + ".offset";
      for (int k = 0; k < last_; ++k)
        if (o.usesDim[k]) pos += " + x" + std::to_string(k) + " * (I)" + r + ".stride[" + std::to_string(k) + "]";
      const bool outerGather = o.gatherDim >= 0 && o.gatherDim != last_;
      if (outerGather) {
        line(d, cll + "g" + u + " = ld_" + typeTag(o.gatherType) + "(" + r + ".index, x" +
                    std::to_string(o.gatherDim) + ");");
        line(d, cb + "bad" + u + " = g" + u + " < 0 || g" + u + " >= " + r + ".gextent;");
        line(d, "if (bad" + u + " && R.error_flag) *R.error_flag = 1;");
        line(d, cll + "q" + u + " = (long long)(" + pos + ") + (bad" + u + " ? 0 : g" + u + " * " + r +
                    ".gstride);");
      } else {
        line(d, cll + "q" + u + " = (long long)(" + pos + ");");
      }
      if (o.step == Operand::Broadcast && o.gatherDim != last_)
        line(d, cv + "s" + u + " = " + (outerGather ? "bad" + u + " ? " + bad() + " : " : "") + ld(o.type) +
                    "(" + r + ".base, q" + u + ");");
    }
  }

  // Operand values for the U groups of this pass; returns the value name.
  Value emitRead(const Operand &o, int d) {
    const std::string u = id(o), r = in(o), tag = typeTag(o.type);
    Value v;
    if (o.step == Operand::Broadcast && o.gatherDim != last_) {
      v.name = "s" + u;
      v.scalar = true;
      return v;
    }
    v.name = "v" + u;
    if (!hoisted_) line(d, ct() + " v" + u + "[U][W];");
    if (o.tiled) {
      unroll();
      line(d, "for (int u = 0; u < U; ++u)");
      unroll();
      line(d + 1, "for (int e = 0; e < W; ++e)");
      line(d + 2, "v" + u + "[u][e] = e < nvalid[u] ? tile[" + std::to_string(o.tileSlot) +
                      "][((int)(j0[u] - tile_q) + e) * PITCH + pl] : " + zero() + ";");
      return v;
    }
    const std::string nan = bad();
    if (o.gatherDim == last_) {
      // one index per element.  Branch-free: every index is requested, then every element (at
      // index 0 where the index is out of range, at the row's last position where the lane
      // has none), then selects -- loads under branches would be issued one at a time
      line(d, "{");
      line(d + 1, std::string("const long long step = ") +
                      (o.step == Operand::Broadcast ? "0" : r + ".stride[" + std::to_string(last_) + "]") + ";");
      line(d + 1, "long long gi[U][W];");
      unroll();
      line(d + 1, "for (int u = 0; u < U; ++u)");
      unroll();
      line(d + 2, "for (int e = 0; e < W; ++e)");
      line(d + 3, "gi[u][e] = ld_" + std::string(typeTag(o.gatherType)) + "(" + r + ".index, (long long)(e < nvalid[u] ? j0[u] + e : n - 1));");
      if (requestHere_ && stage_ && &o == &operands_[stageOperand_])
        line(d + 1, "request(row + rblocks * rows_per_pass < rows ? row + rblocks * rows_per_pass : row);   // the next row's source, see above");
      line(d + 1, "bool any_bad = false;");
      unroll();
      line(d + 1, "for (int u = 0; u < U; ++u)");
      unroll();
      line(d + 2, "for (int e = 0; e < W; ++e) {");
      line(d + 3, "const bool bad = gi[u][e] < 0 || gi[u][e] >= " + r + ".gextent;");
      line(d + 3, "any_bad = any_bad || (bad && e < nvalid[u]);");
      if (stage_ && &o == &operands_[stageOperand_])
        line(d + 3, "const " + ct() + " x = " + std::string(integer_ ? "staged_" : "stage_") + tag + "(sbase + (bad ? 0 : gi[u][e]));");
      else
        line(d + 3, "const " + ct() + " x = " + ld(o.type) + "(" + r + ".base, q" + u +
                        " + (long long)(e < nvalid[u] ? j0[u] + e : n - 1) * step + (bad ? 0 : gi[u][e]) * " + r + ".gstride);");
      line(d + 3, "v" + u + "[u][e] = e < nvalid[u] ? (bad ? " + nan + " : x) : " + zero() + ";");
      line(d + 2, "}");
      line(d + 1, "if (any_bad && R.error_flag) *R.error_flag = 1;");
      line(d, "}");
      return v;
    }
    const bool outerGather = o.gatherDim >= 0;
    const std::string nt = o.readOnce ? "true" : "false";
    if (o.step == Operand::Contiguous) {
      unroll();
      line(d, "for (int u = 0; u < U; ++u) {");
      if (elem_) {
        line(d + 1, "if (false) {");
      } else {
        // aligned kernels: no branch around the load (an empty group reads the row's first
        // vector and drops it), so that nothing is waited for before its use
        line(d + 1, "if (A || V) {");
        line(d + 2, "ldv_" + tag + "<W, " + nt + ">(" + r + ".base, q" + u + " + (A || full[u] ? j0[u] : (I)0), v" + u + "[u]);");
        unroll();
        line(d + 2, "for (int e = 0; e < W; ++e) v" + u + "[u][e] = A || full[u] ? v" + u + "[u][e] : " + zero() + ";");
        line(d + 1, "} else if (full[u] && vec" + u + ") {");
        line(d + 2, "ldv_" + tag + "<W, " + nt + ">(" + r + ".base, q" + u + " + j0[u], v" + u + "[u]);");
      }
      line(d + 1, "} else {");
      unroll();
      // unconditional loads (of the row's last element where the lane has none), then a select:
      // a load under a branch would be waited for before the next one is issued
      line(d + 2, "for (int e = 0; e < W; ++e) v" + u + "[u][e] = " + ld(o.type) + "(" + r + ".base, q" + u +
                      " + (e < nvalid[u] ? j0[u] + e : n - 1));");
      unroll();
      line(d + 2, "for (int e = 0; e < W; ++e) v" + u + "[u][e] = e < nvalid[u] ? v" + u + "[u][e] : " + zero() + ";");
      line(d + 1, "}");
      line(d, "}");
    } else {
      // the stride along the innermost dim is a launch argument; a stride of
      // one (a trailing extent of 1) still takes the 128-bit path
      line(d, "{");
      line(d + 1, "const long long step = " + r + ".stride[" + std::to_string(last_) + "];");
      unroll();
      line(d + 1, "for (int u = 0; u < U; ++u) {");
      if (elem_) line(d + 2, "if (false) {");
      else line(d + 2, "if (step == 1 && (A || (full[u] && (V || vec" + u + ")))) {");
      if (!elem_) line(d + 3, "ldv_" + tag + "<W, " + nt + ">(" + r + ".base, q" + u + " + j0[u], v" + u + "[u]);");
      line(d + 2, "} else {");
      unroll();
      line(d + 3, "for (int e = 0; e < W; ++e) v" + u + "[u][e] = " + ld(o.type) + "(" + r + ".base, q" + u +
                      " + (long long)(e < nvalid[u] ? j0[u] + e : n - 1) * step);");
      unroll();
      line(d + 3, "for (int e = 0; e < W; ++e) v" + u + "[u][e] = e < nvalid[u] ? v" + u + "[u][e] : " + zero() + ";");
      line(d + 2, "}");
      line(d + 1, "}");
      line(d, "}");
    }
    if (outerGather) {
      // a select per element, not a branch around the fill: a branch would make the
      // loads that follow wait for the ones before it
      unroll();
      line(d, "for (int u = 0; u < U; ++u)");
      unroll();
      line(d + 1, "for (int e = 0; e < W; ++e) v" + u + "[u][e] = bad" + u + " ? " + nan + " : v" + u + "[u][e];");
    }
    return v;
  }

  // The expression for the U groups of this pass; returns the value to store.
  Value emitExpression(int d) { return emitCompute(d, emitReads(d)); }

  // Every operand is requested before the first use of any.
  std::vector<Value> emitReads(int d) {
    std::vector<Value> read(operands_.size());
    std::vector<bool> have(operands_.size(), false);
    int push = 0;
    for (const Op &op : seg_.ops)
      if (op.code == OpCode::Push) {
        const int k = pushSlot_[push++];
        if (stage_ && k == stageOperand_) continue;   // last, below
        if (!have[k]) {
          if (!(keepRowConstants_ && rowConstant(operands_[k]))) read[k] = emitRead(operands_[k], d);
          have[k] = true;
        }
      }
    if (stage_) read[stageOperand_] = emitRead(operands_[stageOperand_], d);
    return read;
  }

  // Variables of the row invariants and the operand values, for code that fills them for
  // the next row before it is done with the current one (hoisted_).
  void emitOperandDeclarations(int d) {
    for (int k = 0; k < rank_ - 1; ++k) line(d, "I x" + std::to_string(k) + " = 0;");
    for (const Operand &o : operands_) {
      const std::string u = id(o);
      line(d, "long long q" + u + " = 0;");
      if (o.gatherDim >= 0 && o.gatherDim != last_) {
        line(d, "long long g" + u + " = 0;");
        line(d, "bool bad" + u + " = false;");
      }
      if (o.step == Operand::Broadcast && o.gatherDim != last_) line(d, ct() + " s" + u + " = " + zero() + ";");
      else line(d, ct() + " v" + u + "[U][W];");
    }
  }

  Value emitCompute(int d, const std::vector<Value> &read) {
    std::vector<Value> stack;
    int push = 0, temp = 0, extent = 0;
    auto fresh = [&](bool scalar) {
      Value v;
      v.name = "t" + std::to_string(temp++);
      v.scalar = scalar;
      return v;
    };
    auto define = [&](const Value &v, const std::string &expr) {
      if (v.scalar) {
        line(d, "const " + ct() + " " + v.name + " = " + expr + ";");
      } else {
        line(d, ct() + " " + v.name + "[U][W];");
        unroll();
        line(d, "for (int u = 0; u < U; ++u)");
        unroll();
        line(d + 1, "for (int e = 0; e < W; ++e) " + v.name + "[u][e] = " + expr + ";");
      }
    };
    for (const Op &op : seg_.ops) {
      if (op.code == OpCode::ReduceSum) break;   // what follows works on the row's sum: tailExpression
      switch (op.code) {
        case OpCode::Push:
          stack.push_back(read[pushSlot_[push++]]);
          break;
        case OpCode::Const: {
          Value v = fresh(true);
          // an extent is known at the launch, not here: it arrives with the arguments
          if (op.extent) define(v, "R.extent_const[" + std::to_string(extent++) + "]");
          else define(v, integer_ ? intLiteral(op.constant) : floatLiteral(op.constant));
          stack.push_back(v);
          break;
        }
        case OpCode::Dup:
          stack.push_back(stack[stack.size() - 1 - op.depth]);
          break;
        case OpCode::Add: case OpCode::Sub: case OpCode::Mul: case OpCode::Div:
        case OpCode::Max: case OpCode::Min: {
          const Value b = stack.back();
          stack.pop_back();
          const Value a = stack.back();
          stack.pop_back();
          Value v = fresh(a.scalar && b.scalar);
          std::string expr;
          if (integer_) {
            // wrapping 32-bit arithmetic: through unsigned, where overflow is defined
            // an i16 region compares the low 16 bits; add, sub, mul agree modulo 2^16 anyway
            const std::string ua = "(unsigned)" + a.at(), ub = "(unsigned)" + b.at();
            const std::string ca = narrow_ ? "(int)(short)" + a.at() : a.at(), cb = narrow_ ? "(int)(short)" + b.at() : b.at();
            switch (op.code) {
              case OpCode::Add: expr = "(int)(" + ua + " + " + ub + ")"; break;
              case OpCode::Sub: expr = "(int)(" + ua + " - " + ub + ")"; break;
              case OpCode::Mul: expr = "(int)(" + ua + " * " + ub + ")"; break;
              case OpCode::Max: expr = ca + " > " + cb + " ? " + ca + " : " + cb; break;
              default: expr = ca + " < " + cb + " ? " + ca + " : " + cb; break;
            }
          } else
          switch (op.code) {
            case OpCode::Add: expr = a.at() + " + " + b.at(); break;
            case OpCode::Sub: expr = a.at() + " - " + b.at(); break;
            case OpCode::Mul: expr = a.at() + " * " + b.at(); break;
            case OpCode::Div: expr = a.at() + " / " + b.at(); break;
            case OpCode::Max: expr = "fmax_ieee(" + a.at() + ", " + b.at() + ")"; break;
            default: expr = "fmin_ieee(" + a.at() + ", " + b.at() + ")"; break;
          }
          define(v, expr);
          stack.push_back(v);
          break;
        }
        case OpCode::Cast: {
          const Value a = stack.back();
          stack.pop_back();
          Value v = fresh(a.scalar);
          define(v, std::string("rt_") + typeTag(op.constType) + "(" + a.at() + ")");
          stack.push_back(v);
          break;
        }
        case OpCode::Relu: case OpCode::Leaky: case OpCode::Neg: {
          const Value a = stack.back();
          stack.pop_back();
          Value v = fresh(a.scalar);
          if (integer_) {
            const std::string ca = narrow_ ? "(int)(short)" + a.at() : a.at();
            define(v, op.code == OpCode::Relu ? ca + " > 0 ? " + ca + " : 0" : "(int)(0u - (unsigned)" + a.at() + ")");
          }
          else if (op.code == OpCode::Relu) define(v, "fmax_ieee(" + a.at() + ", 0.f)");
          else if (op.code == OpCode::Leaky)
            define(v, "fmax_ieee(" + a.at() + ", " + a.at() + " * " + floatLiteral(op.constant) + ")");
          else define(v, "-" + a.at());
          stack.push_back(v);
          break;
        }
        case OpCode::ReduceSum: case OpCode::Store: case OpCode::Matmul:
          break;
      }
    }
    return stack.back();
  }

  // The operations after 'reduce sum' as a C expression in the row's sum `s`: constants are
  // literals, extent constants R.extent_const[k], k counting the segment's extent constants in
  // program order (those before 'reduce sum' come first).  `s` itself when there are none.
  std::string tailExpression(const std::string &s) const {
    std::vector<std::string> stack;
    bool after = false;
    int extent = 0;
    for (const Op &op : seg_.ops) {
      if (op.code == OpCode::ReduceSum) {
        after = true;
        stack.assign(1, s);
        continue;
      }
      if (!after && op.code == OpCode::Const && op.extent) ++extent;
      if (!after || op.code == OpCode::Store) continue;
      switch (op.code) {
        case OpCode::Const:
          stack.push_back(op.extent ? "R.extent_const[" + std::to_string(extent++) + "]" : floatLiteral(op.constant));
          break;
        case OpCode::Dup:
          stack.push_back(stack[stack.size() - 1 - op.depth]);
          break;
        case OpCode::Relu: stack.back() = "fmax_ieee(" + stack.back() + ", 0.f)"; break;
        case OpCode::Leaky:
          stack.back() = "fmax_ieee(" + stack.back() + ", (" + stack.back() + ") * " + floatLiteral(op.constant) + ")";
          break;
        case OpCode::Neg: stack.back() = "(-" + stack.back() + ")"; break;
        case OpCode::Cast: stack.back() = std::string("rt_") + typeTag(op.constType) + "(" + stack.back() + ")"; break;
        default: {
          const std::string b = stack.back();
          stack.pop_back();
          const std::string a = stack.back();
          switch (op.code) {
            case OpCode::Add: stack.back() = "(" + a + " + " + b + ")"; break;
            case OpCode::Sub: stack.back() = "(" + a + " - " + b + ")"; break;
            case OpCode::Mul: stack.back() = "(" + a + " * " + b + ")"; break;
            case OpCode::Div: stack.back() = "(" + a + " / " + b + ")"; break;
            case OpCode::Max: stack.back() = "fmax_ieee(" + a + ", " + b + ")"; break;
            default: stack.back() = "fmin_ieee(" + a + ", " + b + ")"; break;
          }
        }
      }
    }
    return after ? stack.back() : s;
  }

  void emitPositionOfRow(int d, const std::string &row = "row") {
    const std::string ci = hoisted_ ? "" : "const I ";
    if (rank_ == 2) {
      line(d, ci + "x0 = " + row + ";");
    } else if (rank_ == 3) {
      line(d, ci + "x0 = sizeof(I) == 4 ? (I)((unsigned)" + row + " / (unsigned)R.size[1]) : (I)(" + row + " / (I)R.size[1]);");
      line(d, ci + "x1 = " + row + " - x0 * (I)R.size[1];");
    }
  }

  // j0 / nvalid / full of the U groups of a pass that starts at group `first`
  // with `lanes` lanes on the row.
  void emitGroups(int d, const std::string &first, const std::string &lanes, const std::string &base = "") {
    line(d, "I j0[U];");
    line(d, "int nvalid[U];");
    line(d, "bool full[U];");
    unroll();
    line(d, "for (int u = 0; u < U; ++u) {");
    line(d + 1, "j0[u] = " + (base.empty() ? std::string() : base + " + ") + "(" + first + " + (I)u * " + lanes + ") * W;");
    line(d + 1, "const I left = n - j0[u];");
    line(d + 1, "nvalid[u] = (A || left >= W) ? W : (V ? 0 : (left > 0 ? (int)left : 0));");
    line(d + 1, "full[u] = A || nvalid[u] == W;");
    line(d, "}");
  }

  void emitBody() {
    const std::string otag = typeTag(p_.output().type);
    os_ << "\n// ---- segment " << index_ << ": iteration rank " << rank_
        << (reduce_ ? ", row sum over the innermost dim" : ", parallel") << "; a lane takes " << U_
        << (U_ == 1 ? " group of " : " groups of ") << W_ << " elements per pass"
        << (slim_ ? " (for rows of few groups)" : elem_ ? " (for unaligned rows)"
                  : stageWave_ ? " (a wavefront per row, the gathered operand's source row staged in LDS)"
                  : stage_ ? " (a workgroup per row, the gathered operand's source row staged in LDS)" : "") << " ----\n";
    os_ << "// I: position type.  M: 2 = every 128-bit access is aligned and every pass is whole (no tail);\n";
    os_ << "// 1 = aligned and the innermost extent a multiple of W, passes may be partly empty; 0 = anything.\n";
    os_ << "template <typename I, int M>\nDEV void segment" << index_ << (slim_ ? "_slim" : elem_ ? "_elem" : stageWave_ ? "_stagew" : stage_ ? "_stage" : "")
        << "(const SpecArgs &R, const I bid, const I nblocks) {\n";
    line(1, "constexpr int W = " + std::to_string(W_) + ", U = " + std::to_string(U_) + ";");
    line(1, "constexpr bool A = M == 2, V = M >= 1;");
    line(1, "const int tid = (int)__builtin_amdgcn_workitem_id_x();");
    line(1, "const I n = (I)R.size[" + std::to_string(last_) + "];");
    line(1, "const I groups = (n + (W - 1)) / W;");
    if (rank_ == 1) line(1, "const I rows = 1;");
    else if (rank_ == 2) line(1, "const I rows = (I)R.size[0];");
    else line(1, "const I rows = (I)(R.size[0] * R.size[1]);");
    for (const Operand &o : operands_)
      if (o.step != Operand::Broadcast && o.gatherDim != last_)
        line(1, "const bool vec" + id(o) + " = " + in(o) + ".vec != 0" + (o.gatherDim >= 0 ? " && " + in(o) + ".gvec != 0" : "") + ";");
    if (reduce_) {
      line(1, "// 2^lanes_log2 (at most 64) lanes of a wavefront share a row: short rows get several rows per wavefront");
      line(1, "const int lane = tid & 63;");
      line(1, "const I lanes = (I)1 << R.lanes_log2;");
      line(1, "const I rows_per_wave = (I)(64 >> R.lanes_log2);");
      line(1, "const I wave = bid * 4 + (I)(tid >> 6);");
      line(1, "const I nwaves = nblocks * 4;");
      line(1, "for (I row0 = wave * rows_per_wave; row0 < rows; row0 += nwaves * rows_per_wave) {");
      line(2, "const I row = row0 + (I)(lane >> R.lanes_log2);");
      line(2, "if (row >= rows) continue;");
      emitPositionOfRow(2);
      emitRowInvariants(2);
      line(2, "float acc[U][W];");
      unroll();
      line(2, "for (int u = 0; u < U; ++u)");
      unroll();
      line(3, "for (int e = 0; e < W; ++e) acc[u][e] = 0.f;");
      line(2, "for (I first = (I)lane & (lanes - 1); first < groups; first += lanes * U) {");
      emitGroups(3, "first", "lanes");
      const Value v = emitExpression(3);
      unroll();
      line(3, "for (int u = 0; u < U; ++u)");
      unroll();
      line(4, "for (int e = 0; e < W; ++e) acc[u][e] += (e < nvalid[u]) ? " + v.at() + " : 0.f;");
      line(2, "}");
      line(2, "// fixed-order combination: groups, then element slots pairwise, then the wavefront");
      unroll();
      line(2, "for (int w = U / 2; w >= 1; w >>= 1)");
      unroll();
      line(3, "for (int u = 0; u < w; ++u)");
      unroll();
      line(4, "for (int e = 0; e < W; ++e) acc[u][e] = acc[2 * u][e] + acc[2 * u + 1][e];");
      unroll();
      line(2, "for (int w = W / 2; w >= 1; w >>= 1)");
      unroll();
      line(3, "for (int e = 0; e < w; ++e) acc[0][e] = acc[0][2 * e] + acc[0][2 * e + 1];");
      line(2, "const float s = R.lanes_log2 == 6 ? wave_sum(acc[0][0]) : lanes_sum(acc[0][0], lane, (int)lanes);");
      line(2, "if ((lane & ((int)lanes - 1)) == 0) st_" + otag + "(R.out, (long long)row, " + tailExpression("s") + ");");
      line(1, "}");
      os_ << "}\n";
      return;
    }
    if (stage_) {
      if (stageWave_) {
        line(1, "// every wavefront walks rows of its own: its accesses to its part of the LDS are ordered, no barriers");
        line(1, "const int sl = tid & 63;   // lane of the row's lane set");
        line(1, "const I lanes = 64, rows_per_pass = 4, local_row = (I)(tid >> 6), first_group = (I)sl;");
        line(1, "const long long sbase = (long long)(tid >> 6) * " + in(operands_[stageOperand_]) + ".gextent;");
      } else {
        line(1, "// the workgroup walks one row at a time");
        line(1, "const int sl = tid;");
        line(1, "const I lanes = 256, rows_per_pass = 1, local_row = 0, first_group = (I)tid;");
        line(1, "const long long sbase = 0;");
      }
      line(1, "constexpr int SL = " + std::string(stageWave_ ? "64" : "256") + ";   // lanes that share a row");
      line(1, "const I cblocks = 1, rblocks = nblocks, cbid = 0, rbid = bid;");
      {
        // A source row of at most PF * 256 chunks is requested one row ahead, into registers.
        // The request follows the index loads of the row's first pass and precedes their first
        // use, in straight-line code: loads return in order, so the wait for the indices leaves
        // the younger request in flight while the row is gathered.  (Rows that are longer, and
        // the last row, still issue the PF loads: a branch around them would make the compiler
        // wait for everything at the join.)
        const Operand &so = operands_[stageOperand_];
        const int epv = 16 / (int)elemTypeBytes(so.type);
        const char *ctype = elemTypeBytes(so.type) == 2 ? "unsigned short" : "unsigned";
        line(1, "constexpr int PF = 4;");
        line(1, "const I chunks = (I)(" + in(so) + ".gextent / " + std::to_string(epv) + ");");
        line(1, "const bool ahead = chunks <= (I)(PF * SL);");
        line(1, "__attribute__((address_space(3))) u32x4 *const srow = (__attribute__((address_space(3))) u32x4 *)afir_stage + (sbase / " +
                    std::to_string(epv) + ");");
        line(1, "u32x4 nx[PF];");
        line(1, "auto request = [&](const I r) {   // chunks past the row's end: chunk 0 again, never stored");
        line(2, "const u32x4 *src = (const u32x4 *)((const " + std::string(ctype) + " *)" + in(so) + ".base + (long long)((I)" +
                    in(so) + ".offset + r * (I)" + in(so) + ".stride[0]));");
        unroll();
        line(2, "for (int k = 0; k < PF; ++k) nx[k] = ld128<false>(src + ((I)sl + (I)(k * SL) < chunks ? (I)sl + (I)(k * SL) : (I)0));");
        line(1, "};");
        line(1, "request(rbid * rows_per_pass + local_row < rows ? rbid * rows_per_pass + local_row : (I)0);");
      }
    } else {
    line(1, "const I lanes = (I)1 << R.lanes_log2;");
    line(1, "const I rows_per_pass = (I)(256 >> R.lanes_log2);");
    line(1, "const I local_row = (I)(tid >> R.lanes_log2);");
    line(1, "const I first_group = (I)tid & (lanes - 1);");
    line(1, "// few, long rows: column_blocks workgroups share a pass of rows, each taking every column_blocks-th stretch");
    line(1, "const I cblocks = (I)R.column_blocks, rblocks = cblocks == 1 ? nblocks : nblocks / cblocks;");
    line(1, "const I cbid = cblocks == 1 ? (I)0 : bid / rblocks, rbid = bid - cbid * rblocks;");
    }
    line(1, "for (I row0 = rbid * rows_per_pass; row0 < rows; row0 += rblocks * rows_per_pass) {");
    line(2, "const I row = row0 + local_row;");
    line(2, "if (row >= rows) continue;");
    emitPositionOfRow(2);
    emitRowInvariants(2);
    if (stage_) {
      const Operand &so = operands_[stageOperand_];
      const char *ctype = elemTypeBytes(so.type) == 2 ? "unsigned short" : "unsigned";
      line(2, "{  // the source row of operand " + id(so) + ": " + in(so) + ".gextent elements, 128-bit loads into LDS");
      line(3, "if (ahead) {");
      unroll();
      line(4, "for (int k = 0; k < PF; ++k)");
      line(5, "if ((I)sl + (I)(k * SL) < chunks) srow[sl + k * SL] = nx[k];");
      line(3, "} else {");
      line(4, "const u32x4 *src = (const u32x4 *)((const " + std::string(ctype) + " *)" + in(so) + ".base + q" + id(so) + ");");
      line(4, "for (I c = (I)sl; c < chunks; c += SL)");
      line(5, "srow[c] = ld128<false>(src + c);");
      line(3, "}");
      line(2, "}");
      line(2, "__builtin_amdgcn_fence(__ATOMIC_RELEASE, \"workgroup\");");
      if (!stageWave_) line(2, "__builtin_amdgcn_s_barrier();");
      line(2, "__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, \"workgroup\");");
    }
    // one pass of the lanes over the row, for the groups that start at `first`
    auto emitPass = [&]() {
      emitGroups(3, "first", "lanes");
      const Value v = emitExpression(3);
      std::string res = v.name;
      if (v.scalar) {
        line(3, ct() + " splat[U][W];");
        unroll();
        line(3, "for (int u = 0; u < U; ++u)");
        unroll();
        line(4, "for (int e = 0; e < W; ++e) splat[u][e] = " + v.name + ";");
        res = "splat";
      }
      unroll();
      line(3, "for (int u = 0; u < U; ++u) {");
      line(4, "const long long o = (long long)row * (long long)n + (long long)j0[u];");
      if (elem_) line(4, "if (false) {");
      else line(4, "if (A || (full[u] && (V || R.out_vec))) {");
      if (!elem_) line(5, "stv_" + otag + "<W>(R.out, o, " + res + "[u]);");
      line(4, "} else if (!V) {");
      unroll();
      line(5, "for (int e = 0; e < W; ++e)");
      line(6, "if (e < nvalid[u]) st_" + otag + "(R.out, o + e, " + res + "[u][e]);");
      line(4, "}");
      line(3, "}");
    };
    if (stage_) {
      // the row's first pass, taken by every lane (a lane past the row's end has empty groups:
      // these kernels run where the innermost extent is a multiple of W), requests the next row
      line(2, "{");
      line(3, "const I first = first_group;");
      requestHere_ = true;
      emitPass();
      requestHere_ = false;
      line(2, "}");
      line(2, "for (I first = first_group + lanes * U; first < groups; first += lanes * U) {");
    } else {
      line(2, "for (I first = first_group + cbid * lanes * U; first < groups; first += cblocks * lanes * U) {");
    }
    emitPass();
    line(2, "}");
    if (stage_ && !stageWave_) line(2, "__builtin_amdgcn_s_barrier();   // the staged row is replaced by the next one");
    line(1, "}");
    os_ << "}\n";
  }

  // The form that separates the chip's reads from its writes in time (specPhased).  HBM serves
  // a pure read stream and a pure write stream faster than their mixture, so a launch whose
  // lanes are all resident at once first requests everything, computes as the loads arrive,
  // keeps the packed results in registers, and stores once the chip's reads have been served:
  // R.hold_ticks of the real-time counter after the workgroup started (a time, so that no
  // workgroup has to hear from another).  The hold shapes the timing only.
  void emitBodyPhased() {
    const std::string otag = typeTag(p_.output().type);
    const int wideU = U_;
    const int G = kSpecPhasedGroups, rounds = phased_.streamed;
    U_ = G / rounds;
    os_ << "\n// ---- segment " << index_ << ", reads and writes separated in time: every lane of the launch resident at once,\n"
        << "// " << G << " groups of " << W_ << " elements per lane in " << rounds << (rounds == 1 ? " round" : " rounds")
        << ", the packed results held in registers until the chip's reads are done ----\n";
    os_ << "template <typename I>\nDEV void segment" << index_ << "_phased(const SpecArgs &R, const I bid, const int place, const int nblocks) {\n";
    line(1, "constexpr int W = " + std::to_string(W_) + ", G = " + std::to_string(G) + ", U = " + std::to_string(U_) + ";");
    line(1, "constexpr bool A = true, V = true;");
    line(1, "const long long t_start = (long long)__builtin_readsteadycounter();");
    line(1, "const int tid = (int)__builtin_amdgcn_workitem_id_x();");
    line(1, "const I n = (I)R.size[" + std::to_string(last_) + "];");
    for (const Operand &o : operands_)
      if (o.step != Operand::Broadcast)
        line(1, "const bool vec" + id(o) + " = true;");
    line(1, "const I lanes = (I)1 << R.lanes_log2;");
    line(1, "const I rows_per_block = (I)(256 >> R.lanes_log2);");
    line(1, "// rows of more than a workgroup's 2048 groups: column_blocks workgroups per row, a stretch each");
    line(1, "const I cblocks = (I)R.column_blocks;");
    line(1, "const I rb = cblocks == 1 ? bid : bid / cblocks, cb = bid - rb * cblocks;");
    line(1, "const I row = rb * rows_per_block + (I)(tid >> R.lanes_log2);");
    line(1, "const I first_group = cb * (I)(256 * G) + ((I)tid & (lanes - 1));");
    emitPositionOfRow(1);
    emitRowInvariants(1);
    line(1, "u32x4 res[G];");
    if (phased_.vectors) {
      line(1, "// the row vectors, 16-byte chunks: [vector][chunk of the row]");
      line(1, "__attribute__((address_space(3))) u32x4 *const rowvec = (__attribute__((address_space(3))) u32x4 *)afir_stage;");
      line(1, "const int row_chunks = (int)(n / W);");
    }
    for (int r = 0; r < rounds; ++r) {
      line(1, "{   // round " + std::to_string(r));
      line(2, "const I first = first_group + (I)" + std::to_string(r * U_) + " * lanes;");
      emitGroups(2, "first", "lanes");
      // every load of the round is issued as a raw 16-byte chunk before anything is converted;
      // the groups are then converted, computed and packed one at a time, so that the round
      // needs the registers of its chunks and of one group's values, not of all of them
      std::vector<Value> read(operands_.size());
      for (size_t k = 0; k < operands_.size(); ++k) {
        const Operand &o = operands_[k];
        if (o.phase == Operand::PhaseScalar) {
          read[k].name = "s" + id(o);
          read[k].scalar = true;
        } else if (o.phase == Operand::PhaseStreamed) {
          const std::string u = id(o), es = std::to_string(elemTypeBytes(o.type));
          line(2, "u32x4 raw" + u + "[U];");
          unroll();
          line(2, "for (int u = 0; u < U; ++u)");
          line(3, "raw" + u + "[u] = ld128<" + (o.readOnce ? "true" : "false") + ">((const u32x4 *)((const char *)" + in(o) +
                      ".base + (q" + u + " + (long long)j0[u]) * " + es + "));");
        }
      }
      if (r == 0 && phased_.vectors) {
        line(2, "// behind the row loads: the row vectors into LDS, once per workgroup");
        for (const Operand &o : operands_)
          if (o.phase == Operand::PhaseVector) {
            const std::string es = std::to_string(elemTypeBytes(o.type));
            line(2, "for (int c = tid; c < row_chunks; c += 256)");
            line(3, "rowvec[" + std::to_string(o.vectorSlot) + " * row_chunks + c] = ld128<false>((const u32x4 *)((const char *)" +
                        in(o) + ".base + " + in(o) + ".offset * " + es + ") + c);");
          }
        line(2, "__builtin_amdgcn_fence(__ATOMIC_RELEASE, \"workgroup\");");
        line(2, "__builtin_amdgcn_s_barrier();");
        line(2, "__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, \"workgroup\");");
      }
      unroll();
      line(2, "for (int g = 0; g < " + std::to_string(U_) + "; ++g) {");
      line(3, "constexpr int U = 1;   // one group at a time from here on");
      for (size_t k = 0; k < operands_.size(); ++k) {
        const Operand &o = operands_[k];
        if (o.phase == Operand::PhaseScalar) continue;
        const std::string u = id(o), tag = typeTag(o.type);
        line(3, ct() + " v" + u + "[U][W];");
        if (o.phase == Operand::PhaseStreamed) {
          line(3, "cvt_" + tag + "(raw" + u + "[g], v" + u + "[0]);");
          if (o.gatherDim >= 0) {
            unroll();
            line(3, "for (int e = 0; e < W; ++e) v" + u + "[0][e] = bad" + u + " ? " + bad() + " : v" + u + "[0][e];");
          }
        } else {
          line(3, "cvt_" + tag + "(rowvec[" + std::to_string(o.vectorSlot) + " * row_chunks + (int)(j0[g] / W)], v" + u + "[0]);");
        }
        read[k].name = "v" + u;
        read[k].scalar = false;
      }
      const Value v = emitCompute(3, read);
      if (v.scalar) {
        line(3, ct() + " splat[W];");
        unroll();
        line(3, "for (int e = 0; e < W; ++e) splat[e] = " + v.name + ";");
        line(3, "res[" + std::to_string(r * U_) + " + g] = pk_" + otag + "(splat);");
      } else {
        line(3, "res[" + std::to_string(r * U_) + " + g] = pk_" + otag + "(" + v.name + "[0]);");
      }
      line(2, "}");
      line(1, "}");
    }
    line(1, "// the results exist here, so the wait for the loads sits before the hold");
    unroll();
    line(1, "for (int g = 0; g < G; ++g) asm volatile(\"\" : \"+v\"(res[g]));");
    line(1, "{");
    line(2, "// A workgroup whose own loads came back early can tell from its place in the launch when the");
    line(2, "// last workgroup's will (the chip serves a one-wave launch in the order of its workgroups):");
    line(2, "// it waits for the shorter of that estimate and the launch's hold.");
    line(2, "int hold = R.hold_ticks;");
    line(2, "const int waited = (int)((long long)__builtin_readsteadycounter() - t_start);");
    line(2, "const float over = waited > 80 ? (float)(waited - 80) : 0.f;");
    line(2, "const float estimate = 80.f + over * (float)nblocks / (float)(place + 1);");
    line(2, "if (estimate < (float)hold) hold = (int)estimate;");
    line(2, "for (int spin = 0; spin < (1 << 15) && (long long)__builtin_readsteadycounter() - t_start < hold; ++spin)");
    line(3, "__builtin_amdgcn_s_sleep(1);");
    line(1, "}");
    line(1, "u32x4 *const out_row = (u32x4 *)R.out + ((long long)row * (long long)n) / W;");
    unroll();
    line(1, "for (int g = 0; g < G; ++g) __builtin_nontemporal_store(res[g], out_row + (first_group + (I)g * lanes));");
    os_ << "}\n";
    U_ = wideU;
  }

  // Row sums of rows of exactly 256 * U groups, every access 128-bit: a
  // workgroup owns a row (lane t takes the groups t, t + 256, ...), so the grid
  // walks the operands like a linear stream, and the operands of the
  // workgroup's next row are requested before the current row is reduced.
  // Partial sums of the four wavefronts meet in LDS, double-buffered by row
  // parity: one barrier per row.  Measured 5 % above a wavefront per row on
  // 8192 rows of 4096 floats; rows of 256 * U / 2 groups measured the same on
  // both and stay with a wavefront per row.
  void emitBodyRowGroup() {
    const std::string otag = typeTag(p_.output().type);
    os_ << "\n// ---- segment " << index_ << ", rows of exactly " << 256 * U_ * W_
        << " elements: a workgroup per row, the next row in flight ----\n";
    os_ << "template <typename I>\nDEV void segment" << index_
        << "_rows(const SpecArgs &R, const I bid, const I nblocks) {\n";
    line(1, "constexpr int W = " + std::to_string(W_) + ", U = " + std::to_string(U_) + ";");
    line(1, "constexpr bool A = true, V = true;");
    line(1, "__attribute__((shared)) static float part[2][4];");
    line(1, "const int tid = (int)__builtin_amdgcn_workitem_id_x();");
    line(1, "const int lane = tid & 63, wave = tid >> 6;");
    line(1, "const I n = (I)R.size[" + std::to_string(last_) + "];");
    if (rank_ == 2) line(1, "const I rows = (I)R.size[0];");
    else line(1, "const I rows = (I)(R.size[0] * R.size[1]);");
    for (const Operand &o : operands_)
      if (o.step != Operand::Broadcast && o.gatherDim != last_)
        line(1, "const bool vec" + id(o) + " = " + in(o) + ".vec != 0" + (o.gatherDim >= 0 ? " && " + in(o) + ".gvec != 0" : "") + ";");
    emitGroups(1, "(I)tid", "(I)256");
    hoisted_ = true;
    emitOperandDeclarations(1);
    line(1, "I row = bid;");
    line(1, "if (row < rows) {");
    emitPositionOfRow(2);
    emitRowInvariants(2);
    const std::vector<Value> read = emitReads(2);
    line(1, "}");
    line(1, "int parity = 0;");
    line(1, "for (; row < rows; row += nblocks) {");
    const Value v = emitCompute(2, read);
    line(2, "float acc[W];");
    unroll();
    line(2, "for (int e = 0; e < W; ++e) {");
    line(3, "float t[U];");
    unroll();
    line(3, "for (int u = 0; u < U; ++u) t[u] = (e < nvalid[u]) ? " + v.at() + " : 0.f;");
    unroll();
    line(3, "for (int w = U / 2; w >= 1; w >>= 1)");
    unroll();
    line(4, "for (int u = 0; u < w; ++u) t[u] = t[2 * u] + t[2 * u + 1];");
    line(3, "acc[e] = t[0];");
    line(2, "}");
    line(2, "const I next = row + nblocks;");
    line(2, "if (next < rows) {");
    emitPositionOfRow(3, "next");
    keepRowConstants_ = true;     // what does not depend on the row stays in its registers
    emitRowInvariants(3);
    emitReads(3);
    keepRowConstants_ = false;
    line(2, "}");
    unroll();
    line(2, "for (int w = W / 2; w >= 1; w >>= 1)");
    unroll();
    line(3, "for (int e = 0; e < w; ++e) acc[e] = acc[2 * e] + acc[2 * e + 1];");
    line(2, "const float s = wave_sum(acc[0]);");
    line(2, "if (lane == 0) part[parity][wave] = s;");
    line(2, "__builtin_amdgcn_fence(__ATOMIC_RELEASE, \"workgroup\");");
    line(2, "__builtin_amdgcn_s_barrier();");
    line(2, "__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, \"workgroup\");");
    line(2, "if (tid == 0) {");
    line(3, "const float s = (part[parity][0] + part[parity][1]) + (part[parity][2] + part[parity][3]);");
    line(3, "st_" + otag + "(R.out, (long long)row, " + tailExpression("s") + ");");
    line(2, "}");
    line(2, "parity ^= 1;");
    line(1, "}");
    os_ << "}\n";
    hoisted_ = false;
  }

  // Row sums of a few long rows (a whole number of passes of 256 * U groups): a
  // workgroup per row again, walking the row pass by pass with the next pass
  // (of this row or of the workgroup's next row) in flight; the lane's partial
  // sums run over the passes and meet as above when the row ends.  A wavefront
  // per row would leave most of the chip idle when there are few rows.
  void emitBodyLongRows() {
    const std::string otag = typeTag(p_.output().type);
    os_ << "\n// ---- segment " << index_ << ", few rows of a multiple of " << 256 * U_ * W_
        << " elements: a workgroup per row, the next pass in flight ----\n";
    os_ << "template <typename I>\nDEV void segment" << index_
        << "_long(const SpecArgs &R, const I bid, const I nblocks) {\n";
    line(1, "constexpr int W = " + std::to_string(W_) + ", U = " + std::to_string(U_) + ";");
    line(1, "constexpr bool A = true, V = true;");
    line(1, "__attribute__((shared)) static float part[2][4];");
    line(1, "const int tid = (int)__builtin_amdgcn_workitem_id_x();");
    line(1, "const int lane = tid & 63, wave = tid >> 6;");
    line(1, "const I n = (I)R.size[" + std::to_string(last_) + "];");
    line(1, "const I passes = n / (I)(256 * U * W);");
    if (rank_ == 2) line(1, "const I rows = (I)R.size[0];");
    else line(1, "const I rows = (I)(R.size[0] * R.size[1]);");
    for (const Operand &o : operands_)
      if (o.step != Operand::Broadcast && o.gatherDim != last_)
        line(1, "const bool vec" + id(o) + " = " + in(o) + ".vec != 0" + (o.gatherDim >= 0 ? " && " + in(o) + ".gvec != 0" : "") + ";");
    line(1, "I j0[U];");
    line(1, "int nvalid[U];");
    line(1, "bool full[U];");
    unroll();
    line(1, "for (int u = 0; u < U; ++u) {");
    line(2, "j0[u] = ((I)tid + (I)u * (I)256) * W;");
    line(2, "nvalid[u] = W;");
    line(2, "full[u] = true;");
    line(1, "}");
    hoisted_ = true;
    emitOperandDeclarations(1);
    line(1, "I row = bid, pass = 0;");
    line(1, "if (row < rows) {");
    emitPositionOfRow(2);
    emitRowInvariants(2);
    const std::vector<Value> read = emitReads(2);
    line(1, "}");
    line(1, "int parity = 0;");
    line(1, "float acc[W];");
    unroll();
    line(1, "for (int e = 0; e < W; ++e) acc[e] = 0.f;");
    line(1, "while (row < rows) {");
    const Value v = emitCompute(2, read);
    unroll();
    line(2, "for (int e = 0; e < W; ++e) {");
    line(3, "float t[U];");
    unroll();
    line(3, "for (int u = 0; u < U; ++u) t[u] = " + v.at() + ";");
    unroll();
    line(3, "for (int w = U / 2; w >= 1; w >>= 1)");
    unroll();
    line(4, "for (int u = 0; u < w; ++u) t[u] = t[2 * u] + t[2 * u + 1];");
    line(3, "acc[e] += t[0];");
    line(2, "}");
    line(2, "const bool row_ends = pass + 1 == passes;");
    line(2, "const I next_row = row_ends ? row + nblocks : row;");
    line(2, "const I next_pass = row_ends ? (I)0 : pass + 1;");
    line(2, "if (next_row < rows) {");
    unroll();
    line(3, "for (int u = 0; u < U; ++u) j0[u] = ((I)tid + (I)u * (I)256 + next_pass * (I)(256 * U)) * W;");
    emitPositionOfRow(3, "next_row");
    emitRowInvariants(3);
    emitReads(3);
    line(2, "}");
    line(2, "if (row_ends) {");
    unroll();
    line(3, "for (int w = W / 2; w >= 1; w >>= 1)");
    unroll();
    line(4, "for (int e = 0; e < w; ++e) acc[e] = acc[2 * e] + acc[2 * e + 1];");
    line(3, "const float s = wave_sum(acc[0]);");
    line(3, "if (lane == 0) part[parity][wave] = s;");
    line(3, "__builtin_amdgcn_fence(__ATOMIC_RELEASE, \"workgroup\");");
    line(3, "__builtin_amdgcn_s_barrier();");
    line(3, "__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, \"workgroup\");");
    line(3, "if (tid == 0) {");
    line(4, "const float s = (part[parity][0] + part[parity][1]) + (part[parity][2] + part[parity][3]);");
    line(4, "st_" + otag + "(R.out, (long long)row, " + tailExpression("s") + ");");
    line(3, "}");
    line(3, "parity ^= 1;");
    unroll();
    line(3, "for (int e = 0; e < W; ++e) acc[e] = 0.f;");
    line(2, "}");
    line(2, "row = next_row;");
    line(2, "pass = next_pass;");
    line(1, "}");
    os_ << "}\n";
    hoisted_ = false;
  }

  // Row sums of a handful of very long rows, in two launches: `column_blocks`
  // workgroups per row each sum a stretch of whole passes (the next pass in
  // flight) and leave one float in afir_region_partials; then a wavefront per
  // row adds the row's partial sums in a fixed order.  Deterministic, and the
  // whole chip works on a single row if that is all there is.  The partial
  // sums live in the code object: launches of one code object that overlap on
  // different streams would share them.
  void emitBodySplitRows() {
    const std::string otag = typeTag(p_.output().type);
    os_ << "\n// ---- segment " << index_ << ", a handful of rows of a multiple of " << 256 * U_ * W_
        << " elements: several workgroups per row, then a join ----\n";
    os_ << "template <typename I>\nDEV void segment" << index_
        << "_split(const SpecArgs &R, const I bid, const I nblocks) {\n";
    line(1, "constexpr int W = " + std::to_string(W_) + ", U = " + std::to_string(U_) + ";");
    line(1, "constexpr bool A = true, V = true;");
    line(1, "__attribute__((shared)) static float part[4];");
    line(1, "const int tid = (int)__builtin_amdgcn_workitem_id_x();");
    line(1, "const int lane = tid & 63, wave = tid >> 6;");
    line(1, "const I n = (I)R.size[" + std::to_string(last_) + "];");
    line(1, "const I passes = n / (I)(256 * U * W);");
    line(1, "const I cblocks = (I)R.column_blocks;");
    line(1, "const I row = bid / cblocks, cb = bid - row * cblocks;");
    line(1, "const I per_block = (passes + cblocks - 1) / cblocks;");
    line(1, "const I first_pass = cb * per_block;");
    line(1, "const I end_pass = first_pass + per_block < passes ? first_pass + per_block : passes;");
    line(1, "(void)nblocks;");
    for (const Operand &o : operands_)
      if (o.step != Operand::Broadcast && o.gatherDim != last_)
        line(1, "const bool vec" + id(o) + " = " + in(o) + ".vec != 0" + (o.gatherDim >= 0 ? " && " + in(o) + ".gvec != 0" : "") + ";");
    line(1, "I j0[U];");
    line(1, "int nvalid[U];");
    line(1, "bool full[U];");
    unroll();
    line(1, "for (int u = 0; u < U; ++u) {");
    line(2, "j0[u] = ((I)tid + (I)u * (I)256 + first_pass * (I)(256 * U)) * W;");
    line(2, "nvalid[u] = W;");
    line(2, "full[u] = true;");
    line(1, "}");
    hoisted_ = true;
    emitOperandDeclarations(1);
    emitPositionOfRow(1);
    emitRowInvariants(1);
    line(1, "float acc[W];");
    unroll();
    line(1, "for (int e = 0; e < W; ++e) acc[e] = 0.f;");
    line(1, "if (first_pass < end_pass) {");
    const std::vector<Value> read = emitReads(2);
    line(1, "}");
    line(1, "for (I pass = first_pass; pass < end_pass; ++pass) {");
    const Value v = emitCompute(2, read);
    unroll();
    line(2, "for (int e = 0; e < W; ++e) {");
    line(3, "float t[U];");
    unroll();
    line(3, "for (int u = 0; u < U; ++u) t[u] = " + v.at() + ";");
    unroll();
    line(3, "for (int w = U / 2; w >= 1; w >>= 1)");
    unroll();
    line(4, "for (int u = 0; u < w; ++u) t[u] = t[2 * u] + t[2 * u + 1];");
    line(3, "acc[e] += t[0];");
    line(2, "}");
    line(2, "if (pass + 1 < end_pass) {");
    unroll();
    line(3, "for (int u = 0; u < U; ++u) j0[u] += (I)(256 * U * W);");
    keepRowConstants_ = false;
    emitReads(3);
    line(2, "}");
    line(1, "}");
    unroll();
    line(1, "for (int w = W / 2; w >= 1; w >>= 1)");
    unroll();
    line(2, "for (int e = 0; e < w; ++e) acc[e] = acc[2 * e] + acc[2 * e + 1];");
    line(1, "const float s = wave_sum(acc[0]);");
    line(1, "if (lane == 0) part[wave] = s;");
    line(1, "__builtin_amdgcn_fence(__ATOMIC_RELEASE, \"workgroup\");");
    line(1, "__builtin_amdgcn_s_barrier();");
    line(1, "__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, \"workgroup\");");
    line(1, "if (tid == 0) afir_region_partials[(long long)row * (long long)cblocks + (long long)cb] = (part[0] + part[1]) + (part[2] + part[3]);");
    os_ << "}\n";
    hoisted_ = false;
    os_ << "template <typename I>\nDEV void segment" << index_
        << "_join(const SpecArgs &R, const I bid, const I nblocks) {\n";
    line(1, "const int tid = (int)__builtin_amdgcn_workitem_id_x();");
    line(1, "const int lane = tid & 63;");
    if (rank_ == 2) line(1, "const I rows = (I)R.size[0];");
    else line(1, "const I rows = (I)(R.size[0] * R.size[1]);");
    line(1, "const I cblocks = (I)R.column_blocks;");
    line(1, "(void)nblocks;");
    line(1, "const I row = bid * 4 + (I)(tid >> 6);");
    line(1, "if (row >= rows) return;");
    line(1, "float s = 0.f;");
    line(1, "for (I c = (I)lane; c < cblocks; c += 64) s += afir_region_partials[(long long)row * (long long)cblocks + (long long)c];");
    line(1, "s = wave_sum(s);");
    line(1, "if (lane == 0) st_" + otag + "(R.out, (long long)row, " + tailExpression("s") + ");");
    os_ << "}\n";
  }

  // Parallel segment with transposed reads: a workgroup takes a tile of kTileP
  // (the dim those operands are contiguous along) x kTileQ (the innermost
  // iteration dim).  Phase 1 loads each transposed operand's tile with 128-bit
  // loads along ITS contiguous dim and writes it to LDS as float32, rows padded
  // by one word; phase 2 is the ordinary row code, 8 lanes per row, reading
  // those operands from LDS column-wise (at most two lanes per bank with the odd pitch).
  void emitBodyTiled() {
    const std::string otag = typeTag(p_.output().type);
    const int p = tileDim_, r = rank_ == 3 ? (p == 0 ? 1 : 0) : -1;
    const std::string P = std::to_string(p), L = std::to_string(last_);
    const int kTileP = opt_.tileP, kTileQ = opt_.tileQ;
    os_ << "\n// ---- segment " << index_ << ": iteration rank " << rank_ << ", parallel, tiles of " << kTileP
        << " (dim " << p << ") x " << kTileQ << " (dim " << last_ << ") through LDS; a lane takes " << U_
        << " groups of " << W_ << " elements per row ----\n";
    os_ << "// I: position type.  A: every 128-bit access is aligned and every tile is whole.\n";
    os_ << "template <typename I, int M>\nDEV void segment" << index_
        << "(const SpecArgs &R, const I bid, const I nblocks) {\n";
    line(1, "constexpr int W = " + std::to_string(W_) + ", U = " + std::to_string(U_) + ";");
    line(1, "constexpr bool A = M == 2, V = false;   // tiles are whole and aligned, or anything goes");
    line(1, "constexpr int TP = " + std::to_string(kTileP) + ", TQ = " + std::to_string(kTileQ) + ", PITCH = TP + 1;");
    line(1, "static_assert(8 * U * W == TQ, \"eight lanes cover a tile row\");");
    line(1, "__attribute__((shared)) static " + ct() + " tile[" + std::to_string(numTiles_) + "][TQ * PITCH];");
    line(1, "const int tid = (int)__builtin_amdgcn_workitem_id_x();");
    line(1, "const I n = (I)R.size[" + L + "];");
    line(1, "const I np = (I)R.size[" + P + "];");
    line(1, "const I tiles_q = (n + (TQ - 1)) / TQ, tiles_p = (np + (TP - 1)) / TP;");
    line(1, std::string("const I ntiles = tiles_q * tiles_p") + (r >= 0 ? " * (I)R.size[" + std::to_string(r) + "]" : "") + ";");
    for (const Operand &o : operands_)
      if (o.step != Operand::Broadcast && o.gatherDim != last_)
        line(1, "const bool vec" + id(o) + " = " + in(o) + ".vec != 0" + (o.gatherDim >= 0 ? " && " + in(o) + ".gvec != 0" : "") + ";");
    line(1, "for (I t = bid; t < ntiles; t += nblocks) {");
    line(2, "const I tq = t % tiles_q, rest = t / tiles_q;");
    line(2, "const I tp = rest % tiles_p;");
    if (r >= 0) line(2, "const I x" + std::to_string(r) + " = rest / tiles_p;");
    line(2, "const I tile_p = tp * TP, tile_q = tq * TQ;");
    for (const Operand &o : operands_) {
      if (!o.tiled) continue;
      const std::string u = id(o), rr = in(o), tag = typeTag(o.type);
      const int el = (o.type == ElemType::F32 || o.type == ElemType::I32) ? 4 : 8;
      line(2, "{  // operand " + u + ": " + std::to_string(kTileQ) + " runs of " + std::to_string(kTileP) + " elements along dim " + P);
      line(3, "constexpr int EL = " + std::to_string(el) + ", LPR = TP / EL, RPP = 256 / LPR, NP = TQ / RPP;");
      line(3, "const int lp = (tid % LPR) * EL, lq = tid / LPR;");
      line(3, "const long long pos = (long long)" + rr + ".offset" +
                  (r >= 0 && o.usesDim[r] ? " + (long long)x" + std::to_string(r) + " * " + rr + ".stride[" + std::to_string(r) + "]" : "") +
                  " + (long long)(tile_p + lp);");
      line(3, "const long long sq = " + rr + ".stride[" + L + "];");
      line(3, ct() + " vals[NP][EL];");
      unroll();
      line(3, "for (int s = 0; s < NP; ++s) {");
      line(4, "const I q = tile_q + (I)(lq + s * RPP);");
      line(4, "if (A || (vec" + u + " && q < n && tile_p + (I)(lp + EL) <= np)) {");
      line(5, "ldv_" + tag + "<EL, " + (o.readOnce ? "true" : "false") + ">(" + rr + ".base, pos + (long long)q * sq, vals[s]);");
      line(4, "} else {");
      line(5, "// unconditional loads, of the last element inside where the position is outside, then a select");
      line(5, "const I qc = q < n ? q : n - 1;");
      unroll();
      line(5, "for (int e = 0; e < EL; ++e)");
      line(6, "vals[s][e] = " + ld(o.type) + "(" + rr + ".base, pos + (long long)qc * sq + (tile_p + (I)(lp + e) < np ? (long long)e : (long long)(np - 1) - (long long)(tile_p + (I)lp)));");
      unroll();
      line(5, "for (int e = 0; e < EL; ++e)");
      line(6, "vals[s][e] = (q < n && tile_p + (I)(lp + e) < np) ? vals[s][e] : " + zero() + ";");
      line(4, "}");
      line(3, "}");
      unroll();
      line(3, "for (int s = 0; s < NP; ++s)");
      unroll();
      line(4, "for (int e = 0; e < EL; ++e) tile[" + std::to_string(o.tileSlot) + "][(lq + s * RPP) * PITCH + lp + e] = vals[s][e];");
      line(2, "}");
    }
    line(2, "__builtin_amdgcn_fence(__ATOMIC_RELEASE, \"workgroup\");");
    line(2, "__builtin_amdgcn_s_barrier();");
    line(2, "__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, \"workgroup\");");
    unroll();
    line(2, "for (int pp = 0; pp < TP / 32; ++pp) {");
    line(3, "const int pl = (tid >> 3) + 32 * pp;");
    line(3, "const I x" + P + " = tile_p + (I)pl;");
    line(3, "if (A || x" + P + " < np) {");
    if (rank_ == 2) line(4, "const I row = x0;");
    else line(4, "const I row = x0 * (I)R.size[1] + x1;");
    emitRowInvariants(4);
    emitGroups(4, "(I)(tid & 7)", "(I)8", "tile_q");
    const Value v = emitExpression(4);
    std::string res = v.name;
    if (v.scalar) {
      line(4, ct() + " splat[U][W];");
      unroll();
      line(4, "for (int u = 0; u < U; ++u)");
      unroll();
      line(5, "for (int e = 0; e < W; ++e) splat[u][e] = " + v.name + ";");
      res = "splat";
    }
    unroll();
    line(4, "for (int u = 0; u < U; ++u) {");
    line(5, "const long long o = (long long)row * (long long)n + (long long)j0[u];");
    line(5, "if (A || (full[u] && R.out_vec)) {");
    line(6, "stv_" + otag + "<W>(R.out, o, " + res + "[u]);");
    line(5, "} else {");
    unroll();
    line(6, "for (int e = 0; e < W; ++e)");
    line(7, "if (e < nvalid[u]) st_" + otag + "(R.out, o + e, " + res + "[u][e]);");
    line(5, "}");
    line(4, "}");
    line(3, "}");
    line(2, "}");
    line(2, "__builtin_amdgcn_s_barrier();   // the tile is reused by the next iteration");
    line(1, "}");
    os_ << "}\n";
  }

  void emitWrappers() {
    for (int i32 = 1; i32 >= 0; --i32)
      for (int mode = kSpecAligned; mode >= kSpecGeneral; --mode) {
        if (mode == kSpecVector && tiled()) continue;   // tiles are whole and aligned, or general
        os_ << "KERNEL void " << specKernelName(index_, i32 != 0, mode) << "(const SpecArgs R) { segment" << index_
            << "<" << (i32 ? "int" : "long long") << ", " << mode
            << ">(R, (" << (i32 ? "int" : "long long") << ")__builtin_amdgcn_workgroup_id_x(), ("
            << (i32 ? "int" : "long long") << ")R.grid); }\n";
      }
    if (phased_.eligible)
      os_ << "PHASED_KERNEL void " << specPhasedKernelName(index_) << "(const SpecArgs R) { segment" << index_
          << "_phased<int>(R, (int)__builtin_amdgcn_workgroup_id_x() + R.first_block, (int)__builtin_amdgcn_workgroup_id_x(), R.grid); }\n";
    if (!tiled())
      for (int i32 = 1; i32 >= 0; --i32)
        os_ << "KERNEL void " << specElementKernelName(index_, i32 != 0) << "(const SpecArgs R) { segment" << index_
            << "_elem<" << (i32 ? "int" : "long long") << ", 0>(R, (" << (i32 ? "int" : "long long")
            << ")__builtin_amdgcn_workgroup_id_x(), (" << (i32 ? "int" : "long long") << ")R.grid); }\n";
    if (stageOperand_ >= 0)
      for (int wave = 0; wave < 2; ++wave)
        for (int i32 = 1; i32 >= 0; --i32)
          for (int mode = kSpecAligned; mode >= kSpecVector; --mode)
            os_ << "KERNEL void " << specStagedKernelName(index_, i32 != 0, mode, wave != 0) << "(const SpecArgs R) { segment"
                << index_ << (wave ? "_stagew<" : "_stage<") << (i32 ? "int" : "long long") << ", " << mode << ">(R, ("
                << (i32 ? "int" : "long long") << ")__builtin_amdgcn_workgroup_id_x(), (" << (i32 ? "int" : "long long")
                << ")R.grid); }\n";
    if (hasSlim_)
      for (int mode = kSpecAligned; mode >= kSpecVector; --mode)
        os_ << "KERNEL void " << specSlimKernelName(index_, mode) << "(const SpecArgs R) { segment" << index_
            << "_slim<int, " << mode << ">(R, (int)__builtin_amdgcn_workgroup_id_x(), (int)R.grid); }\n";
    if (reduce_)
      for (int i32 = 1; i32 >= 0; --i32)
        os_ << "KERNEL void " << specRowsKernelName(index_, i32 != 0) << "(const SpecArgs R) { segment" << index_
            << "_rows<" << (i32 ? "int" : "long long")
            << ">(R, (" << (i32 ? "int" : "long long") << ")__builtin_amdgcn_workgroup_id_x(), ("
            << (i32 ? "int" : "long long") << ")R.grid); }\n";
    if (reduce_)
      for (int i32 = 1; i32 >= 0; --i32)
        for (int join = 0; join < 2; ++join)
          os_ << "KERNEL void " << specSplitRowsKernelName(index_, i32 != 0, join != 0) << "(const SpecArgs R) { segment"
              << index_ << (join ? "_join<" : "_split<") << (i32 ? "int" : "long long")
              << ">(R, (" << (i32 ? "int" : "long long") << ")__builtin_amdgcn_workgroup_id_x(), ("
              << (i32 ? "int" : "long long") << ")R.grid); }\n";
    if (reduce_)
      for (int i32 = 1; i32 >= 0; --i32)
        os_ << "KERNEL void " << specLongRowsKernelName(index_, i32 != 0) << "(const SpecArgs R) { segment" << index_
            << "_long<" << (i32 ? "int" : "long long")
            << ">(R, (" << (i32 ? "int" : "long long") << ")__builtin_amdgcn_workgroup_id_x(), ("
            << (i32 ? "int" : "long long") << ")R.grid); }\n";
  }

  const Program &p_;
  const Segment &seg_;
  int index_;
  std::ostringstream &os_;
  EmitOptions opt_;
  int rank_ = 0, last_ = 0, W_ = 8, U_ = 2;
  int tileDim_ = -1, numTiles_ = 0;
  bool reduce_ = false;
  bool integer_ = false;   // 32-bit integers instead of float32 values
  bool narrow_ = false;    // ... of which the low 16 bits are the value (i16 output)
  bool slim_ = false;      // emitting the one-group-per-lane form of the segment
  bool elem_ = false;      // emitting the one-element-per-group form (no 128-bit accesses)
  bool stage_ = false;     // emitting the form that stages the gathered operand's source row in LDS
  bool requestHere_ = false;   // ... and the pass that requests the next row's source
  bool stageWave_ = false;     // ... with a wavefront per row (four rows per workgroup, no barriers)
  int stageOperand_ = -1;  // index into operands_ of that operand, else -1
  bool hasSlim_ = false;   // ... which exists for this segment
  bool hoisted_ = false;   // row invariants and operand values are assigned, not declared
  bool keepRowConstants_ = false;   // ... and operands that are the same for every row are left alone
  SpecPhased phased_;      // the form that separates reads from writes, if the segment has one

  bool rowConstant(const Operand &o) const {
    if (o.gatherDim >= 0) return false;
    for (int k = 0; k < last_; ++k)
      if (o.usesDim[k]) return false;
    return true;
  }

  // C type of a value, its zero, what an out-of-range gather yields, the scalar load of a tensor
  std::string ct() const { return integer_ ? "int" : "float"; }
  std::string zero() const { return integer_ ? "0" : "0.f"; }
  std::string bad() const { return integer_ ? "0" : "as_f32(0x7fc00000u)"; }
  std::string ld(ElemType t) const { return std::string(integer_ ? "ldd_" : "ld_") + typeTag(t); }
  std::vector<Operand> operands_;
  std::vector<int> pushSlot_;   // per push, in order: index into operands_
};

}  // namespace

std::string checkEmitOptions(const EmitOptions &o) {
  if (o.tileP < 32 || o.tileP > 256 || o.tileP % 32 != 0) return "tile_p must be a multiple of 32 in 32..256";
  if (o.tileQ != 64 && o.tileQ != 128 && o.tileQ != 256) return "tile_q must be 64, 128 or 256";
  if ((long long)o.tileQ * (o.tileP + 1) * 4 * kMaxTiles > 160 * 1024) return "tile_p x tile_q does not fit the LDS";
  if (o.unroll != 0 && o.unroll != 1 && o.unroll != 2 && o.unroll != 4 && o.unroll != 8)
    return "unroll must be 0 (by element types), 1, 2, 4 or 8";
  return "";
}

bool setEmitOption(EmitOptions *o, const std::string &name, long long value) {
  if (name == "tile_p") o->tileP = (int)value;
  else if (name == "tile_q") o->tileQ = (int)value;
  else if (name == "unroll") o->unroll = (int)value;
  else return false;
  return true;
}

SpecShape specShape(const Program &p, int segment, const EmitOptions &options) {
  const Segment &g = p.segments[segment];
  bool any16 = false, any32 = false;
  auto note = [&](ElemType t) { (elemTypeBytes(t) == 4 ? any32 : any16) = true; };
  note(p.output().type);
  for (const Op &op : g.ops)
    if (op.code == OpCode::Push) note(p.args[op.arg].type);
  SpecShape s;
  s.width = any16 ? 8 : 4;            // 16 bytes of the narrowest tensor
  s.unroll = options.unroll ? options.unroll : ((any16 && any32) ? 2 : 4);
  return s;
}

SpecTile specTile(const Program &p, int segment) {
  std::ostringstream sink;
  SegmentEmitter e(p, segment, sink);
  e.analyze();
  SpecTile t;
  t.tiled = e.tiled();
  t.dim = e.tileDim();
  t.inputs = e.tiledInputs();
  return t;
}

bool specAllSegments(const Program &p) {
  const int nseg = (int)p.segments.size();
  if (nseg < 2 || nseg > kSpecMaxSegments) return false;
  for (int s = 0; s < nseg; ++s) {
    const Segment &g = p.segments[s];
    if (!g.ops.empty() && g.ops[0].code == OpCode::Matmul) return false;
    if (specTile(p, s).tiled) return false;   // LDS tiles of several segments would add up
  }
  return true;
}

void specExtentConstants(const Program &p, int segment, const std::vector<std::vector<int64_t>> &shapes,
                         float (&out)[kSpecMaxExtentConsts]) {
  for (float &v : out) v = 0.f;
  int n = 0;
  for (const Op &op : p.segments[segment].ops)
    if (op.code == OpCode::Const && op.extent && n < kSpecMaxExtentConsts)
      out[n++] = afir_region::roundThroughType((float)shapes[op.constRef.arg][op.constRef.dim], op.constType);
}

uint64_t programHash(const Program &p) {
  uint64_t h = 0xcbf29ce484222325ull;
  for (unsigned char c : serialize(p)) {
    h ^= c;
    h *= 0x100000001b3ull;
  }
  return h;
}

namespace {
const char *modeSuffix(int mode) { return mode == kSpecAligned ? "_a" : mode == kSpecVector ? "_v" : "_g"; }
}  // namespace

std::string specAllKernelName(bool idx32, int mode) {
  return std::string("afir_region_all") + (idx32 ? "_i32" : "_i64") + modeSuffix(mode);
}

std::string specRowsKernelName(int segment, bool idx32) {
  return "afir_region_s" + std::to_string(segment) + "_rows" + (idx32 ? "_i32" : "_i64");
}

std::string specSplitRowsKernelName(int segment, bool idx32, bool join) {
  return "afir_region_s" + std::to_string(segment) + (join ? "_join" : "_split") + (idx32 ? "_i32" : "_i64");
}

std::string specLongRowsKernelName(int segment, bool idx32) {
  return "afir_region_s" + std::to_string(segment) + "_long" + (idx32 ? "_i32" : "_i64");
}

std::string specStagedKernelName(int segment, bool idx32, int mode, bool wave) {
  return "afir_region_s" + std::to_string(segment) + (wave ? "_stagew" : "_stage") + (idx32 ? "_i32" : "_i64") +
         modeSuffix(mode);
}

SpecPhased specPhased(const Program &p, int segment) {
  const Segment &g = p.segments[segment];
  if (!g.ops.empty() && g.ops[0].code == OpCode::Matmul) return SpecPhased();
  std::ostringstream sink;
  SegmentEmitter e(p, segment, sink);
  e.analyze();
  return e.phased();
}

std::string specPhasedKernelName(int segment) { return "afir_region_s" + std::to_string(segment) + "_phased_i32"; }
std::string specAllPhasedKernelName() { return "afir_region_all_phased_i32"; }

SpecStage specStage(const Program &p, int segment) {
  std::ostringstream sink;
  SegmentEmitter e(p, segment, sink);
  e.analyze();
  SpecStage s;
  s.input = e.stagedSlot();
  s.elemBytes = (int)elemTypeBytes(e.stagedType());
  return s;
}

std::string specElementKernelName(int segment, bool idx32) {
  return "afir_region_s" + std::to_string(segment) + "_elem" + (idx32 ? "_i32" : "_i64");
}

std::string specSlimKernelName(int segment, int mode) {
  return "afir_region_s" + std::to_string(segment) + "_slim_i32" + modeSuffix(mode);
}

std::string specKernelName(int segment, bool idx32, int mode) {
  return "afir_region_s" + std::to_string(segment) + (idx32 ? "_i32" : "_i64") + modeSuffix(mode);
}

std::string emitHipSource(const Program &p, const std::string &title, std::string *source,
                          const EmitOptions &options) {
  if (std::string why = validate(p); !why.empty()) return why;
  if (std::string why = checkEmitOptions(options); !why.empty()) return why;
  std::ostringstream os;
  os << "// HIP kernels for the fused region '" << title << "' (gfx950), generated from this program:\n";
  {
    std::istringstream lines(serialize(p));
    for (std::string line; std::getline(lines, line);) os << "//   " << line << "\n";
  }
  os << "// Build: hipcc --genco --offload-arch=gfx950 -O3 -nogpuinc -ffp-contract=off \\\n"
        "//          -Xclang -target-feature -Xclang -packed-fp32-ops -o region.hsaco region.hip\n";
  os << kPrelude;
  os << "static_assert(sizeof(SpecInput) == " << sizeof(SpecInput) << " && sizeof(SpecArgs) == " << sizeof(SpecArgs)
     << " && __builtin_offsetof(SpecArgs, in) == " << offsetof(SpecArgs, in)
     << " && __builtin_offsetof(SpecInput, vec) == " << offsetof(SpecInput, vec)
     << ", \"launch argument layout differs from the kernel library's\");\n";
  char hash[32];
  std::snprintf(hash, sizeof hash, "0x%016llxull", (unsigned long long)programHash(p));
  os << "extern \"C\" __attribute__((device)) __attribute__((used)) const unsigned long long afir_region_program_hash = " << hash << ";\n";
  os << "extern \"C\" __attribute__((device)) __attribute__((used)) const int afir_region_emit_abi = " << kSpecAbiVersion << ";\n";
  os << "extern \"C\" __attribute__((device)) __attribute__((used)) const int afir_region_emit_options[3] = {"
     << options.tileP << ", " << options.tileQ << ", " << options.unroll << "};   // tile_p, tile_q, unroll\n";
  bool reduces = false;
  for (const Segment &g : p.segments)
    for (const Op &op : g.ops) reduces = reduces || op.code == OpCode::ReduceSum;
  if (reduces)
    os << "// partial row sums of the split / join kernels (shared by the launches of this code object)\n"
       << "__attribute__((device)) float afir_region_partials[" << kSpecPartials << "];\n";
  for (int s = 0; s < (int)p.segments.size(); ++s) {
    SegmentEmitter e(p, s, os, options);
    if (std::string why = e.run(); !why.empty()) return why;
  }
  const int nseg = (int)p.segments.size();
  if (specAllSegments(p)) {
    // every segment in one launch: the workgroups are dealt out segment by segment
    os << "\n// ---- all segments in one launch ----\n";
    os << "struct SpecAll {\n  int first[" << kSpecMaxSegments + 1 << "];   // first workgroup of each segment, then the total\n"
       << "  int pad;\n  SpecArgs seg[" << nseg << "];\n};\n";
    os << "static_assert(__builtin_offsetof(SpecAll, seg) == " << offsetof(SpecAll, seg)
       << ", \"launch argument layout differs from the kernel library's\");\n";
    for (int i32 = 1; i32 >= 0; --i32)
      for (int mode = kSpecAligned; mode >= kSpecGeneral; --mode) {
        const char *I = i32 ? "int" : "long long";
        os << "KERNEL void " << specAllKernelName(i32 != 0, mode) << "(const SpecAll S) {\n";
        os << "  const int b = (int)__builtin_amdgcn_workgroup_id_x();\n";
        for (int k = 0; k < nseg; ++k)
          os << "  " << (k ? "else " : "") << (k + 1 < nseg ? "if (b < S.first[" + std::to_string(k + 1) + "]) " : "")
             << "segment" << k << "<" << I << ", " << mode << ">(S.seg[" << k << "], (" << I
             << ")(b - S.first[" << k << "]), (" << I << ")(S.first[" << k + 1 << "] - S.first[" << k << "]));\n";
        os << "}\n";
      }
    bool every = true;
    for (int k = 0; k < nseg; ++k) every = every && specPhased(p, k).eligible;
    if (every) {
      os << "PHASED_KERNEL void " << specAllPhasedKernelName() << "(const SpecAll S) {\n";
      os << "  const int b = (int)__builtin_amdgcn_workgroup_id_x();\n";
      for (int k = 0; k < nseg; ++k)
        os << "  " << (k ? "else " : "") << (k + 1 < nseg ? "if (b < S.first[" + std::to_string(k + 1) + "]) " : "")
           << "segment" << k << "_phased<int>(S.seg[" << k << "], b - S.first[" << k << "], b, S.first[" << nseg << "]);\n";
      os << "}\n";
    }
  }
  *source = os.str();
  return "";
}

std::string hipccCommandLine(const std::string &sourcePath, const std::string &outputPath) {
  return "hipcc --genco --offload-arch=gfx950 -O3 -nogpuinc -ffp-contract=off -Xclang -target-feature -Xclang "
         "-packed-fp32-ops -o " + outputPath + " " + sourcePath;
}

}  // namespace afir_target
