// The reference's HCCL_ALGO setting, read the way its own parser reads it and mapped onto this library's fold
// orders.  Host code only.
//
// Grammar (reference src/common/alg_parse.cc:120-437, HcclAlgoParser::Parser):
//   config   := segment (';' segment)*
//   segment  := [opType ':'] ( 'not' '(' unit ')' | unit )
//   unit     := executor '{' [item (',' item)*] '}'  |  template          (a bare template means sole{template})
//   item     := ['level' N '='] ( 'not' '(' template ')' | template )
// Names are case-insensitive, underscores in template names are dropped (mesh_chunk = meshchunk), blanks are
// skipped.  opType, executor and template names come from the reference's tables (alg_parse.cc:27-86); anything
// else makes the whole string invalid, and an invalid string is ignored with a warning, as the reference does
// (alg_parse.cc:803-826).
#pragma once

#include <string>
#include <vector>

#include "hccl.h"

namespace hccl_amd {

struct AlgoTemplate {
    std::string name;     // lower case, e.g. "meshconcur"
    bool enable = true;   // false: written as not(name)
};

struct AlgoSegment {
    std::string opType;     // lower case; empty = every operator
    std::string executor;   // "sole", "sequence", "parallel", "pipeline", "concur", "strictordered"
    std::vector<AlgoTemplate> templates;   // by level, ascending
    bool enable = true;     // false: written as not(...)
};

// HCCL_E_PARA for a string the reference's parser rejects; `segments` is then unspecified.
HcclResult ParseHcclAlgo(const std::string& config, std::vector<AlgoSegment>* segments);

// What a parsed configuration selects for the operators whose result depends on the fold order.
struct AlgoSelection {
    bool set[HCCL_AMD_OP_COUNT] = {};
    HcclAmdAlgo algo[HCCL_AMD_OP_COUNT] = {};
    // The configured executor runs a level-0 template inside groups of ranks and `algo` between them
    // (sequence{mesh_concur, rhd} and its relatives); only meaningful where the world has level-0 groups.
    bool twoLevel[HCCL_AMD_OP_COUNT] = {};
};

// Segments are taken last to first and the first one that selects something for an operator settles that
// operator, whether it names the operator or applies to all of them, like the reference's marking pass
// (alg_parse.cc:670-760).  Negated segments and templates only exclude candidates in the reference and select
// nothing here.  Segments for operators without a fold order (the copies) are accepted and ignored.
AlgoSelection SelectFromHcclAlgo(const std::vector<AlgoSegment>& segments);

}  // namespace hccl_amd
