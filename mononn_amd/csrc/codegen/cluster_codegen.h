// Per-node device functions: fused memory-bound clusters (element-wise loops and row programs)
// and GEMMs with their fused epilogues.
//
// Reference counterparts: ClusterElewise / ClusterReduce code shapes
// (mononn_engine/core/op/cluster_elewise.cc:247-348, cluster_reduce.cc:249-497), loop schedules
// T0..T2 (mononn_engine/core/schedule/schedule_factory.cc:29-89), GemmImpl::generate_impl
// (mononn_engine/core/op_impl/gemm_impl.cc:55-141) and ClusterCodegen (codegen/cluster_codegen.cc:37-119).
#pragma once
#include <string>
#include <vector>

#include "codegen/emitter.h"
#include "graph/program.h"

namespace mononn {
namespace codegen {

struct LaunchShape {
  int block_size = 256;   // threads per workgroup (multiple of 64)
  // waves that share a SIMD when the whole grid is resident (grid beyond one workgroup per CU): the register
  // budget of a wave is 512 / waves_per_simd, and the operand chunks of the GEMM tile shrink with it
  int waves_per_simd = 1;
  int waves() const { return block_size / 64; }
  int chunk_fragments() const { return waves_per_simd >= 2 ? 16 : 32; }        // mirrors mononn_dev::gemm_chunk_steps
  int whole_range_fragments() const { return waves_per_simd >= 2 ? 24 : 56; }
};

// per-cluster knobs; names follow the reference's cluster_*_spec fields
// (tuning_space_generator.cc:151-160, :184-194)
struct ClusterTuning {
  int ilp_factor = 1;        // independent elements per thread per trip (element-wise clusters)
  int locality_tier = 1;     // row programs: 1 = one wave per row, 2 = one workgroup per row
  // row programs of tier 1: 0 = a wave on one row; 1 / 2 / 3 = a wave on 8 / 4 / 2 consecutive rows at once, 8 / 16 / 32
  // lanes per row (every load and store instruction then covers whole 128-byte lines of those rows, and one trip
  // moves that many rows' worth of bytes)
  int reduce_implementation = 0;
};

// Regional synchronisation: how the units of a node are dealt to the XCDs.  With parts > 0 unit u belongs to XCD
// u % 8 (units are dealt to the workgroups round-robin and a workgroup's XCD is its index modulo 8); XCD x < parts
// takes partition x of the node's work, XCDs from `parts` on have empty units:
//   kColumns  a GEMM's result columns in `parts` equal slices (all rows, whole k range)
//   kSplitK   the k slices of a GEMM that is split `parts` ways over workgroups
//   kHeads    the batch elements of an attention node in `parts` equal runs
struct Partition {
  enum Kind { kNone, kColumns, kSplitK, kHeads };
  Kind kind = kNone;
  int parts = 0;
  bool on() const { return kind != kNone && parts > 0; }
};

// Where a node writes element (bidx, m, n) of its GEMM-shaped result: the element offset inside the buffer of
// `root`, as the epilogue computes it (through reshapes, transposes and fragment-order layouts)
struct WriteMap {
  const hlo::Instr* root = nullptr;
  LinExpr offset;
  int vb = -1, vm = -1, vm4 = -1, vn4 = -1, vr = -1, vnn = -1;   // variables of `offset`; -1 = not used
  size_t num_vars = 0;
  int64_t batch = 1, M = 0, N = 0;
  // false when the offset has run-time terms
  bool element_offset(int64_t bidx, int64_t m, int64_t n, int64_t* out) const;
};

struct GemmTuning {
  Partition part;            // set by the regional synchronisation plan, not by the specification
  int bm = 32, bn = 32;      // workgroup tile
  int wm = 1, wn = 1, wk = 4;   // wave arrangement; wm*wn*wk == waves per workgroup
  int split_k = 1;              // k range also split over workgroups (fp32 partial sums to memory)
  // the function takes the first chunk of packed weights from registers filled by a companion function
  // (NodeFunction::preload_text) that the kernel calls before it waits at the grid barrier
  bool preload_b = false;
  // 2: operand tiles of bk k each are staged through two LDS buffers, once per workgroup
  // (mononn_dev::gemm_tile_lds; wk must be 1); 1: every wave fetches its own fragments from global memory
  int stages = 1;
  int bk = 32;
};

struct NodeFunction {
  std::string text;                            // device function, name written as @NAME@
  std::vector<PointerTable::Entry> pointers;   // call arguments after `unit`, before `smem`
  int64_t num_units = 0;                       // independent work units (one workgroup each)
  int smem_bytes = 0;
  std::vector<std::string> globals;            // device-global definitions the function needs
  // Optional companion `@NAME@_pre(unit, <pointers>, @NAME@_preb&)`: requests operands that do not depend on
  // the previous stage.  When present, `text` defines the register block type `@NAME@_preb` and takes a trailing
  // `const @NAME@_preb&` after `smem`.
  std::string preload_text;
  std::vector<WriteMap> write_maps;            // GEMM and attention nodes: one entry per result written by the epilogue
};

// fills has_reduce / row_program / rows / row_len
void classify_cluster(const graph::Program& prog, graph::Node& node);

NodeFunction generate_cluster(const graph::Program& prog, const graph::Node& node, const LaunchShape& ls,
                              const ClusterTuning& t);
NodeFunction generate_gemm(const graph::Program& prog, const graph::Node& node, const LaunchShape& ls,
                           const GemmTuning& t);

// key_waves: waves of a workgroup that share one block of 16 query rows by splitting the keys between them
// (0 = as many as the key count allows); the remaining factor of the workgroup's waves takes further row blocks
// preload_weights: an absorbed output projection takes its weight fragments from a companion function
// (NodeFunction::preload_text), as generate_gemm does under GemmTuning::preload_b
// row_blocks: blocks of 16 query rows a wave works through, one after the other, with the keys and values it loaded
// once (a unit then covers 16 * row_blocks * (waves / key_waves) rows of one batch element)
NodeFunction generate_attention(const graph::Program& prog, const graph::Node& node, const LaunchShape& ls, int key_waves = 0,
                                bool preload_weights = false, int row_blocks = 1, Partition part = Partition());
// Element offset, inside the buffer of its storage root, of element e = (bidx * M + m) * K + k of a GEMM operand that is
// stored [batch, M, K] with k minor-most, as an expression in one variable (index 0); false when the operand's
// storage does not have that many elements
bool operand_offset_expr(const graph::Program& prog, const hlo::Instr* operand, int64_t elements, LinExpr* out);
// the input of a row program fused in front of a GEMM whose rows the GEMM loads as its left-operand fragments
const hlo::Instr* prologue_primary(const graph::Program& prog, const std::vector<const hlo::Instr*>& row_members, int64_t M, int64_t K);
// the GEMM `gemm3` reads nothing but the heads that the attention's second GEMM produces, merged by pure data movement
bool can_fuse_out_proj(const graph::Program& prog, const hlo::Instr* gemm2, const graph::GemmDesc& d2,
                       const std::vector<const hlo::Instr*>& epilogue_members, const hlo::Instr* gemm3, const graph::GemmDesc& d3, int heads);
int default_attention_key_waves(const graph::GemmDesc& first_gemm, const LaunchShape& ls);

// allow_lds_tile false: the direct tile with k split over the waves whatever the problem size (a GEMM with a row
// program in front that is not a folded LayerNorm: that program runs on the fragments a wave holds in registers)
GemmTuning default_gemm_tuning(const graph::GemmDesc& g, const LaunchShape& ls, int num_cus, bool allow_lds_tile = true);
// throws Error(kSpecError) when the tile / wave arrangement cannot be generated for this GEMM
void validate_gemm_tuning(const graph::GemmDesc& g, const LaunchShape& ls, const GemmTuning& t, bool has_prologue = false);
bool gemm_uses_mfma(const graph::GemmDesc& g);

// dry runs used by the merge passes
bool can_merge_clusters(const graph::Program& prog, const std::vector<const hlo::Instr*>& producer,
                        const std::vector<const hlo::Instr*>& consumer,
                        const std::vector<const hlo::Instr*>& merged);
bool can_fuse_epilogue(const graph::Program& prog, const std::vector<const hlo::Instr*>& gemm_members,
                       const std::vector<const hlo::Instr*>& cluster_members);

// true when the row program `row_members`, whose product `H` is the [M,K] left operand of a GEMM, is exactly
// LayerNorm over the last dimension of its primary input: (x - mean) * rsqrt(var + eps) * gamma + beta
bool match_prologue_layer_norm(const graph::Program& prog, const std::vector<const hlo::Instr*>& row_members, const hlo::Instr* H, int64_t M,
                               int64_t K, const hlo::Instr** gamma, const hlo::Instr** beta, double* eps);
bool can_fuse_prologue(const graph::Program& prog, const std::vector<const hlo::Instr*>& row_members,
                       const std::vector<const hlo::Instr*>& gemm_members, const graph::GemmDesc& g);

bool can_fuse_attention(const graph::Program& prog, const hlo::Instr* gemm1, const graph::GemmDesc& d1,
                        const std::vector<const hlo::Instr*>& row_members, const hlo::Instr* gemm2, const graph::GemmDesc& d2,
                        const std::vector<const hlo::Instr*>& epilogue_members);

// entry-level values defined by `members` that somebody outside (another instruction or the
// module root) reads, in definition order
std::vector<const hlo::Instr*> external_outputs(const graph::Program& prog, const std::vector<const hlo::Instr*>& members);

}  // namespace codegen
}  // namespace mononn
