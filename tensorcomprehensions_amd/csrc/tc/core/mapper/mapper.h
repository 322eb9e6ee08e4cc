// Box mapper: turns a size-specialised TC function into HIP kernels for CDNA4.
//
// Takes the role of the reference's polyhedral GPU mapper and code generator
// (tc/core/polyhedral/cuda/mapped_scop.cc:978-1097 strategy, :137-200/:385-460 block and thread
// mapping, :253-383 reductions, tighten_launch_bounds.cc:49-81, memory_promotion_heuristic.cc,
// cuda/codegen.cc:833-894) without isl: after range inference every statement iterates over a
// rectangular box with (mostly) affine subscripts, so dependences, footprints, launch bounds and
// guards have closed forms.
//
// Pipeline per TC function:
//   1. statements writing the same tensor over the same box are merged into a *stage* whose
//      running value lives in registers (init, reduction update, point-wise epilogues);
//   2. stages are grouped into kernels while every cross-stage dependence is point-wise in a
//      shared prefix of the left-hand-side indices (that prefix is what blocks iterate over);
//   3. per stage: jointly-contiguous loop dimensions are collapsed, the x-mapped dimension is
//      split into vector lanes, the band [parallel..., reduction...] is tiled, tile loops go to
//      blockIdx (outermost first), point loops to threadIdx (innermost -> x) in whole-wavefront
//      friendly shapes, a reduction can be mapped to threadIdx.x and finished by the wave64
//      reduction library, per-thread point loops are unrolled into register tiles under the
//      unroll budget, read-only operands with reuse are staged through LDS;
//   4. launch bounds are tightened to what the mapping uses; HIP C++ is printed.
#pragma once
#include <array>
#include <map>
#include <string>
#include <vector>

#include "tc/core/hip/hip_mapping_options.h"
#include "tc/core/ir.h"

namespace tc {
namespace mapper {

// One iteration variable of a stage after collapsing / lane splitting.
struct LoopVar {
  std::string name;
  int64_t min = 0, extent = 1;
  bool reduction = false;
  bool vectorLane = false;     // innermost unrolled lanes of the x-mapped variable
  int64_t tile = 1;            // point-loop extent
  int64_t numTiles = 1;
  int blockAxis = -1;          // tile loop distributed over blockIdx.{x,y,z} (cyclically)
  int64_t gridExtent = 1;
  int threadAxis = -1;         // point loop distributed over threadIdx.{x,y,z} (cyclically)
  int64_t perThread = 1;       // point iterations executed by one thread
  bool unrolled = false;       // point loop fully unrolled (register tile)
  bool partial() const { return numTiles * tile != extent; }
};

struct TensorView {
  std::string name;
  ir::ScalarType type;
  std::vector<int64_t> extents;   // possibly with merged dimensions
  bool isOutput = false;
};

// A read-only operand staged in LDS for the duration of one (reduction) tile.
struct Promotion {
  std::string tensor;
  std::string ldsName;
  std::vector<int64_t> extents;      // footprint box, per view dimension
  // Distance in the tensor between neighbouring footprint elements of a dimension: above 1 when
  // every access steps through the dimension in multiples of it (I(j, 2 * i + 1)); elements the
  // computation jumps over are not staged.
  std::vector<int64_t> steps;
  std::vector<int64_t> ldsStrides;   // row-major, pitches padded against bank conflicts
  int64_t elems = 0;                 // LDS elements including padding
  int64_t reuse = 1;                 // accesses per staged element
  bool insideReductionTiles = false;
  // 2: the software pipeline over the reduction tiles alternates between two copies of the
  // array (the next tile is stored while the current one is still being read: one barrier per
  // tile instead of two); `elems` is the size of one copy.
  int buffers = 1;
  // An earlier stage of the kernel staged the very same footprint and nothing has overwritten it:
  // this stage reads that copy (`ldsName` names the earlier stage's array) and copies nothing.
  bool sharedWithEarlierStage = false;
};

// One statement of a stage, rewritten on the stage's variables and tensor views.
struct StageStmt {
  ir::ReduceOp op = ir::ReduceOp::None;
  bool init = false;
  ir::ExprRef rhs;
  std::vector<std::string> redVars;
  ir::ScalarType type;
};

struct StagePlan {
  std::string tensor;                // the written tensor
  std::vector<ir::ExprRef> lhsSubs;  // its subscripts on the stage's variables
  std::vector<StageStmt> stmts;
  std::vector<LoopVar> vars;         // parallel variables (left-hand-side order), then reductions
  int numParallel = 0;
  std::map<std::string, TensorView> views;
  bool threadReduction = false;      // innermost reduction variable mapped to threadIdx.x
  std::vector<Promotion> promotions;
  int64_t accCount = 1;              // register-tile size
  // Matrix-core mapping of a dense contraction `out +=! A * B` (useMfma): parallel variables
  // found only in A form the M side, only in B the N side, the rest are batch; each wavefront
  // computes 16x16 output tiles with v_mfma_f32_16x16x4_f32 over the flattened reduction.
  bool mfma = false;
  std::vector<std::string> mfmaM, mfmaN, mfmaBatch, mfmaK;
  bool mfmaSwapOperands = false;     // the first factor of the product is the N-side operand
  int64_t waves = 1;
  // The stage adds partial sums into its tensor with atomics: its first parallel variable numbers
  // slices of the reduction and is no subscript of the tensor.
  bool atomic = false;
};

struct KernelPlan {
  std::string name;
  std::vector<StagePlan> stages;
  int sharedDepth = 0;               // leading parallel variables looped over at kernel level
  std::array<int64_t, 3> grid{{1, 1, 1}};
  std::array<int64_t, 3> block{{1, 1, 1}};
  int64_t ldsBytes = 0;
};

struct DeviceLimits {
  int64_t ldsBytesPerBlock = 65536;
  int64_t maxThreadsPerBlock = 1024;
  int wavefront = 64;
};

struct MappedProgram {
  std::string source;                 // complete translation unit for hipRTC
  std::vector<KernelPlan> kernels;    // launched in this order
  std::vector<std::string> paramNames;
  std::vector<int64_t> paramValues;   // leading scalar kernel arguments, sorted by name
};

// Throws std::runtime_error (TC_CHECK) on options the mapper cannot honour (empty tiling,
// zero-sized grid or block, block larger than the device allows).
MappedProgram mapToHip(
    const ir::Function& f,
    const HipMappingOptions& options,
    const std::string& specializedName,
    const DeviceLimits& limits = DeviceLimits());

} // namespace mapper
} // namespace tc
