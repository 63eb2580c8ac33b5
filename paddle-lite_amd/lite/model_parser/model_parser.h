// The optimised-model file ("<name>.nb") of the reference's `opt` tool:
//   u16 meta_version | char[16] opt version | u64 topology size | topology
//   (a FlatBuffers ProgramDesc) | parameters
// with the parameters of meta version 2 written one by one
//   u16 0 | u16 0 | u16 6 | u16 count | u32 largest tensor bytes |
//   count x { u32 bytes + 4 | u32 4 | FlatBuffers ParamDesc }
// and those of meta version 1 as one FlatBuffers CombinedParamsDesc up to the
// end of the file (reference: lite/model_parser/model_parser.cc:470-535
// SaveModelNaive, :744-905 LoadModelNaiveFromFile / LoadModelFbsFromFile,
// lite/model_parser/flatbuffers/io.cc:71-148).  A sparse_conv2d op arrives
// with its NonZeroWeights / OcNonZeros / Diffs tensors among the parameters
// and first_ic / flag_semi among its attributes, as the detect pass left them.
#pragma once

#include <set>
#include <string>
#include <vector>

#include "lite/core/program_desc.h"
#include "lite/core/scope.h"

namespace paddle {
namespace lite {

// Version string written into a saved file (16 bytes, zero padded).
std::string version();

// Reads a meta version 1 or 2 file into the scope (host tensors, marked
// persistable) and the program.  Malformed input ends in LOG(FATAL), as
// in the reference; the Try form returns false and the reason instead.
void LoadModelNaiveFromFile(const std::string& filename, Scope* scope, cpp::ProgramDesc* cpp_prog);
void LoadModelNaiveFromMemory(const std::string& model_buffer, Scope* scope, cpp::ProgramDesc* cpp_prog);
bool TryLoadModelNaiveFromMemory(const std::string& model_buffer, Scope* scope, cpp::ProgramDesc* cpp_prog, std::string* error);

// Writes "<model_file>.nb": the program and every parameter of block 0
// (persistable tensor variables, each name once, in name order).  Meta
// version 2 unless the environment variable PADDLE_LITE_MODEL_VERSION1 is set.
void SaveModelNaive(const std::string& model_file, const Scope& exec_scope, const cpp::ProgramDesc& cpp_prog);
std::string SerializeModelNaive(const Scope& exec_scope, const cpp::ProgramDesc& cpp_prog, uint16_t meta_version = 2);

// The Diffs tensor of a sparse_conv2d holds byte distances that include the
// H*W of the op's input at optimisation time (the detect pass multiplies the
// channel distance by it, lite/core/optimizer/mir/sparse_conv_detect_pass.cc:
// 35-91), so a saved model runs at that resolution only.  This rewrites the
// Diffs of every sparse_conv2d of block 0 from the recorded shape of its
// Input variable to new_h * new_w and records the new shape, which makes the
// loaded model usable at another resolution.  Returns the number of ops
// changed; an op whose Input has no static 4-D shape is left alone.
int RebakeSparseConvDiffs(cpp::ProgramDesc* prog, Scope* scope, int64_t new_h, int64_t new_w);

namespace fbs {
// The two FlatBuffers payloads on their own.
std::vector<uint8_t> SerializeProgramDesc(const cpp::ProgramDesc& prog);
void ParseProgramDesc(const uint8_t* data, size_t size, cpp::ProgramDesc* prog);
std::vector<uint8_t> SerializeParamDesc(const std::string& name, const Tensor& tensor);
void ParseParamDesc(const uint8_t* data, size_t size, Scope* scope);
}  // namespace fbs

}  // namespace lite
}  // namespace paddle
