// In-memory form of a fused XLA HLO module and its text parser.
//
// The reference receives an xla::HloModule object from its TensorFlow fork and walks it in
// mononn_engine/parser/ir_parser_fused.cc:319-385; the XLA object model is not available here, so
// this parser reads the HLO *text* form of the same module (the reference's own `from_text`
// entry, ir_parser_fused.cc:259-265, does that through XLA's parser).  Accepted dialect = what
// the reference accepts: static shapes, plain minor-to-major layouts without tiling
// (ir_parser_fused.cc:119,136-139), the dtypes of :68-98, tuple results one level deep (:451-455).
#pragma once
#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <vector>

namespace mononn {
namespace hlo {

enum class DType { kPred, kS8, kS16, kS32, kS64, kU8, kU16, kU32, kU64, kF16, kBF16, kF32, kF64, kTuple, kInvalid };

const char* dtype_name(DType t);          // "f16"
int dtype_bytes(DType t);                 // 2
const char* dtype_ctype(DType t);         // device C type, e.g. "_Float16"
DType dtype_from_name(const std::string& s);
inline bool is_float(DType t) { return t == DType::kF16 || t == DType::kBF16 || t == DType::kF32 || t == DType::kF64; }
inline bool is_half_float(DType t) { return t == DType::kF16 || t == DType::kBF16; }   // 2-byte MFMA operand types

struct Shape {
  DType dtype = DType::kInvalid;
  std::vector<int64_t> dims;
  std::vector<int> minor_to_major;   // as written while parsing; descending (row-major) on everything parse_module returns
  std::vector<Shape> tuple;          // when dtype == kTuple

  bool is_tuple() const { return dtype == DType::kTuple; }
  int rank() const { return static_cast<int>(dims.size()); }
  int64_t num_elements() const {
    int64_t n = 1;
    for (auto d : dims) n *= d;
    return n;
  }
  int64_t byte_size() const { return num_elements() * dtype_bytes(dtype); }
  std::string to_string() const;
  bool same_dims(const Shape& o) const { return dims == o.dims; }
};

struct Computation;

struct GemmConfig {   // backend_config of __cublas$gemm (gemm_impl.cc:182-231)
  double alpha_real = 1, alpha_imag = 0, beta = 0;
  int lhs_contracting = 0, rhs_contracting = 0;
  std::vector<int> lhs_batch, rhs_batch;
  int64_t batch_size = 1, lhs_stride = 0, rhs_stride = 0;
  std::string selected_algorithm;
  // __cublas$lt$matmul only: DEFAULT, BIAS, RELU, GELU, BIAS_RELU, BIAS_GELU (the epilogue enum of the newer call);
  // the parser turns it into a fusion behind the call, after which the field is documentation
  std::string epilogue = "DEFAULT";
};

// __cudnn$convForward (attributes read by ir_parser_fused.cc:749-823, lowering conv_impl.cc:252-324):
// input N,H,W,C, filter K,R,S,C, output N,P,Q,K, symmetric padding, no dilation, one feature group
struct ConvConfig {
  int64_t N = 0, H = 0, W = 0, C = 0, K = 0, R = 0, S = 0, P = 0, Q = 0;
  int64_t stride_h = 1, stride_w = 1, pad_h = 0, pad_w = 0;
  double result_scale = 1;
};

struct Instr {
  std::string name;            // canonical: '.' and '-' replaced by '_' (string_helpers.cc:22-32)
  std::string hlo_name;        // as written in the text
  std::string opcode;
  Shape shape;
  std::vector<Instr*> operands;
  std::map<std::string, std::string> attrs;   // raw attribute text
  Computation* parent = nullptr;
  bool is_root = false;
  int index_in_comp = 0;

  // decoded attributes (valid for the opcodes that use them)
  int64_t parameter_number = -1;
  std::string literal;                 // constant payload text; "{...}" when elided
  bool literal_elided = false;
  std::vector<int64_t> dimensions;     // broadcast / transpose / reduce / concatenate
  Computation* called = nullptr;       // fusion calls= / reduce to_apply=
  std::string fusion_kind;             // kLoop | kInput
  std::string comparison;              // EQ NE LT LE GT GE
  int64_t tuple_index = -1;
  int64_t iota_dimension = -1;
  std::vector<int64_t> slice_starts, slice_limits, slice_strides;
  std::vector<int64_t> pad_low, pad_high, pad_interior;
  std::vector<int64_t> dynamic_slice_sizes;
  std::vector<int64_t> window_size, window_stride, window_pad_low, window_pad_high;   // reduce-window
  // gather
  std::vector<int64_t> offset_dims, collapsed_slice_dims, start_index_map, slice_sizes;
  int64_t index_vector_dim = -1;
  // custom-call
  std::string custom_call_target;
  GemmConfig gemm;
  ConvConfig conv;
  bool is_conv() const { return opcode == "custom-call" && custom_call_target == "__cudnn$convForward"; }
  // a dense contraction with a decoded GemmConfig: the cuBLAS custom call, or a plain `dot` (what a stock XLA
  // prints before its GEMM rewriter has run)
  bool is_gemm() const {
    return (opcode == "custom-call" && (custom_call_target == "__cublas$gemm" || custom_call_target == "__cublas$lt$matmul")) || opcode == "dot";
  }
  // __cublas$lt$matmul written with a (result, workspace) tuple: the call carries the result's array shape and its
  // get-tuple-element 0 aliases it, as with the convolution call
  bool lt_tuple_result = false;

  std::vector<Instr*> users;           // within the same computation
  bool is_scalar_constant() const { return opcode == "constant" && shape.num_elements() == 1 && !literal_elided; }
};

struct Computation {
  std::string name;
  std::string hlo_name;
  std::vector<std::unique_ptr<Instr>> instrs;   // definition order (operands before users)
  std::vector<Instr*> params;
  Instr* root = nullptr;
  bool is_entry = false;
};

struct Module {
  std::string name;
  std::vector<std::unique_ptr<Computation>> computations;
  Computation* entry = nullptr;
  std::map<std::string, Computation*> by_name;   // canonical name
};

// Parse HLO text.  Throws Error(kParseError) on malformed text and Error(kUnsupported) on
// constructs outside the dialect (unknown opcode, dynamic dimension, tiled layout ...).
// Minor-to-major orders other than the descending one are taken out of the module: entry parameters, host-supplied
// constants and results become the row-major arrays their memory holds (dims listed slowest first), with
// transposes to and from logical order next to them and around `bitcast`; those next to a GEMM are folded into
// its contracting dimensions or an exchange of its operands.
std::unique_ptr<Module> parse_module(const std::string& text);

// '.' and '-' -> '_'  (mononn_engine/helpers/string_helpers.cc:22-32)
std::string canonical_name(const std::string& hlo_name);
// leading "cluster_<digits>" of a module name (string_helpers.cc:34-48); throws when absent
std::string module_short_name(const std::string& module_name);

}  // namespace hlo
}  // namespace mononn
