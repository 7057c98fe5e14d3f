// Stage-level program: the HLO entry computation regrouped into work nodes (fused memory-bound
// clusters and GEMMs), layered into barrier-separated stages, with buffers assigned.
//
// Reference counterparts: Graph of Op/ClusterOp built by IRParserFused
// (mononn_engine/parser/ir_parser_fused.cc:319-385, :490-539), ClusteringSingleNodePass,
// MergeDependentPass (merge_dependent_pass.cc:37-191), the BFS-depth barrier placement of
// GlobalSynchronizationEliminationPass (global_synchronization_elimination_pass.cc:32-147) and
// BufferAssignmentPass (:34-98).  The reference inherits buffer offsets from XLA's buffer
// assignment; here they are computed (stage-interval colouring of one temp arena).
#pragma once
#include <cstdint>
#include <map>
#include <memory>
#include <set>
#include <string>
#include <vector>

#include "hlo/hlo.h"

namespace mononn {
namespace graph {

// kAttention: GEMM -> row program over the GEMM's rows -> GEMM, executed by one wave per 16 rows with
// the intermediate matrices kept in registers (members: [gemm1, row members..., gemm2, epilogue members...])
enum class NodeKind { kCluster, kGemm, kAttention };

struct GemmDesc {
  int64_t batch = 1, M = 0, N = 0, K = 0;
  bool f32 = false;          // operands and result are f32 (v_mfma_f32_16x16x4_f32 tiles); otherwise f16 or bf16
  bool bf16 = false;         // operands and result are bf16 (the bf16 forms of the f16 MFMAs; same tiles, same layouts)
  bool a_k_contig = true;    // A stored [.., M, K]; false: [.., K, M]
  bool b_k_contig = false;   // B stored [.., N, K]; false: [.., K, N]
  bool b_packed = false;     // B is a constant that the host stores in MFMA fragment order at upload
  bool a_packed = false;     // A is a value of this kernel that its producer stores in MFMA fragment order
  bool b_tiled = false;      // likewise B (only operands of the fused attention; weights use b_packed)
  int split_k = 1;           // k range split over workgroups, fp32 partial sums as output
  int64_t a_batch_stride = 0, b_batch_stride = 0, d_batch_stride = 0;
  double alpha = 1.0, beta = 0.0;
  bool has_addend = false;
  // Forward convolution seen as a GEMM (implicit GEMM, conv_impl.cc:51): M = N*P*Q output pixels, N = K output
  // channels, K = R*S*C; row m of the left operand is gathered from the N,H,W,C input, the filter K,R,S,C is the
  // k-contiguous right operand, the result N,P,Q,K is row-major [M, N].
  bool is_conv = false;
  hlo::ConvConfig conv;
  // left-operand fragments can be loaded 8 halves at a time: no padding, and every 8-element piece of a row
  // lies inside one contiguous run of S*C input elements at a 16-byte aligned address
  bool conv_fragment_loads() const {
    return is_conv && conv.pad_h == 0 && conv.pad_w == 0 && (conv.S * conv.C) % 8 == 0 && (conv.W * conv.C) % 8 == 0 &&
           (conv.stride_w * conv.C) % 8 == 0 && (conv.N == 1 || (conv.H * conv.W * conv.C) % 8 == 0);
  }
  std::string problem_hash() const;   // dtype+shape key, cf. mononn_module_tuner.cc:386-408
};

// LayerNorm in front of a constant-weight GEMM, folded: with h = (x - mean) * r * gamma + beta per row,
//   h . W = r * (x . (gamma o W) - mean * (gamma^T W)) + beta^T W,
// so the MFMAs run on the raw rows x against weights scaled by gamma once on the host, and the row statistics enter
// in the epilogue as a rank-1 correction with two constant column-sum vectors.
struct LayerNormFold {
  const hlo::Instr* gamma = nullptr;
  const hlo::Instr* beta = nullptr;
  double eps = 0;
  const hlo::Instr* colsum_gamma = nullptr;   // f32[N]: sum over k of gamma[k] * W[k, n], a constant built on the host
  const hlo::Instr* colsum_beta = nullptr;    // f32[N]: sum over k of beta[k] * W[k, n]
  bool on() const { return gamma != nullptr; }
};

struct Node {
  int id = -1;
  std::string name;
  NodeKind kind = NodeKind::kCluster;
  // entry-level instructions realised by this node, in definition order.  For a GEMM node the
  // first member is the custom-call; further members are element-wise clusters fused behind it.
  std::vector<const hlo::Instr*> members;
  std::vector<const hlo::Instr*> inputs;    // storage roots read from memory
  std::vector<const hlo::Instr*> outputs;   // entry-level values written to memory (storage roots)
  int stage = 0;
  // clusters
  bool has_reduce = false;
  bool row_program = false;       // reduces over the minor-most dim, rows handled by a wave / workgroup
  int64_t rows = 0, row_len = 0;
  // GEMM (for kAttention: the first GEMM)
  GemmDesc gemm;
  // kGemm: row program (LayerNorm) applied to the rows of the left operand inside the GEMM; the node
  // with prologue_stores also writes the row program's result for consumers in later stages
  std::vector<const hlo::Instr*> prologue;
  bool prologue_stores = false;
  LayerNormFold ln_fold;          // the prologue is a LayerNorm and is folded into weights and epilogue
  // kAttention: second GEMM and where it sits in `members`
  GemmDesc gemm2;
  size_t gemm2_index = 0;
  // kAttention with the output projection absorbed: a third GEMM (constant weights) applied per batch element
  // (head) to that head's slice of the context; its result leaves the node as one fp32 partial sum per head
  GemmDesc gemm3;
  size_t gemm3_index = 0;   // 0 = none
  int heads = 0;            // batch elements of the attention GEMMs per row of the projected matrix
  const hlo::Instr* gemm_instr() const { return kind == NodeKind::kGemm ? members[0] : nullptr; }
};

struct Buffer {
  enum Kind { kParameter, kConstant, kLiveOut, kTemp };
  Kind kind = kTemp;
  int index = 0;          // parameter number / live-out index / constant ordinal
  int64_t offset = 0;     // within the temp arena
  int64_t bytes = 0;
  int def_stage = 0, last_use_stage = 0;
};

// kPackMfmaB: a [K,N] matrix stored as [ceil(N/16)][K/32][64 lanes][8 halves], lane l holding
// W[k = 32*ks + 8*(l/16) + j][n = 16*nt + l%16], columns beyond N zero-filled.
enum class ConstantTransform { kNone, kPackMfmaB };

struct Program {
  std::unique_ptr<hlo::Module> module;
  std::vector<Node> nodes;                                         // topological, grouped by stage
  std::map<const hlo::Instr*, Buffer> buffers;                     // storage root -> buffer
  std::vector<const hlo::Instr*> parameters;                       // entry parameters in order
  std::vector<const hlo::Instr*> constants;                        // non-scalar entry constants (device buffers)
  std::map<const hlo::Instr*, ConstantTransform> constant_transform;
  // Constants of folded LayerNorms.  A weight matrix [K,N] whose rows are multiplied by a [K] vector before it is laid
  // out for the device, and column-sum vectors f32[N] = sum_k vector[k] * weight[k,n] that exist only as module
  // globals: the host builds them from the payloads of their sources (instructions owned by `synthetic`).
  std::map<const hlo::Instr*, const hlo::Instr*> constant_row_scale;
  struct ColumnSums {
    const hlo::Instr* weight = nullptr;
    const hlo::Instr* vector = nullptr;
  };
  std::map<const hlo::Instr*, ColumnSums> derived_constants;
  std::vector<std::unique_ptr<hlo::Instr>> synthetic;
  // storage roots kept in a permuted physical order: physical dim i = logical dim perm[i]
  // (right-hand GEMM operands produced inside the kernel are stored with k minor-most)
  std::map<const hlo::Instr*, std::vector<int>> physical_perm;
  // Storage roots kept in MFMA operand fragment order.  The buffer is seen as a [rows, K] matrix (the row-major
  // linear index, after `physical_perm` if the root has one, is row * K + k); the 16 rows x 32 k of one MFMA step
  // form one contiguous KiB [lane = g * 16 + row % 16][8 halves] at block (row / 16) * (K / 32) + k / 32, so that
  // a wave loads an operand with one fully coalesced instruction.  Two enumerations of k inside a step:
  //   kRunsOf8:  lane group g holds k % 32 in [8g, 8g + 8)            (operands contracted over their minor dim)
  //   kPairsOf4: lane group g holds k % 32 in {4g..4g+3, 16+4g..+3}   (the order in which a lane of the fused
  //              attention holds its probabilities: the right operand of the second contraction)
  // Every reader and the writer of such a root go through codegen::physical_offset.
  enum class TileOrder { kRunsOf8, kPairsOf4 };
  struct TileLayout {
    int64_t k = 0;
    TileOrder order = TileOrder::kRunsOf8;
  };
  std::map<const hlo::Instr*, TileLayout> physical_tile;
  // GEMM results kept as S fp32 partial sums [S][elements] (split-K); readers add them up
  std::map<const hlo::Instr*, int> split_k;
  // Storage roots whose every reader runs on the XCD that wrote the bytes it reads (an annotation of the code
  // generator's regional synchronisation plan, empty otherwise): their writers use ordinary cached stores, the
  // hand-over stays inside that XCD's L2
  mutable std::set<const hlo::Instr*> regional_roots;
  std::vector<const hlo::Instr*> live_outs;                        // storage roots, root-tuple order
  std::map<const hlo::Instr*, int> producer;                       // storage root -> node id
  int num_stages = 0;
  int64_t temp_bytes = 0;

  // value -> the entry-level instruction whose buffer holds it (follows bitcast / reshape)
  const hlo::Instr* storage_root(const hlo::Instr* v) const;
  const Node* node_of(const hlo::Instr* member) const;
  std::string summary() const;
};

struct BuildOptions {
  bool merge_dependent = true;          // glue producer/consumer clusters that share a row space
  bool fuse_gemm_epilogue = true;       // element-wise consumers of a GEMM run in its epilogue
  bool transpose_constant_b = true;     // store constant [K,N] GEMM operands in MFMA fragment order
  bool fuse_gemm_prologue = false;      // row programs feeding a GEMM's left operand run inside that GEMM
  bool fold_layer_norm = false;         // ... and when that row program is a LayerNorm and the weights are constant: folded
  bool fuse_attention = true;           // GEMM -> soft-max style row program -> GEMM in one stage
  bool assign_operand_layouts = true;   // store in-kernel right-hand GEMM operands k-contiguous
  bool pack_left_operands = true;       // store in-kernel left-hand GEMM operands in MFMA fragment order
  // the GEMM that consumes the merged heads of an attention node runs inside that node, head by head; its
  // bias / residual epilogue moves into the consuming row program together with the sum over the heads
  bool fuse_attention_out_proj = false;
  std::map<std::string, int> gemm_split_k;   // GEMM instruction (canonical name) -> k split over workgroups
  bool reuse_temp_slots = true;         // false: every temp value gets its own address (written once per launch)
  std::set<std::string> disabled_passes;   // MONONN_OPTIMIZATION_DISABLED_PASS (config.cc:82-86)
};

// Takes ownership of the module.  Throws Error(kUnsupported) for graphs outside the dialect.
std::unique_ptr<Program> build_program(std::unique_ptr<hlo::Module> module, const BuildOptions& opt);

// true for entry-level instructions that only rename storage (no code): bitcast, reshape
bool is_alias_op(const hlo::Instr* ins);

}  // namespace graph
}  // namespace mononn
