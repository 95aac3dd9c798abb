// Policy index tables of lc0, generated from their closed forms instead of
// being stored: src/neural/tables/attention_policy_map.h:24 (kAttnPolicyMap),
// :386 (kPosEncoding) and src/neural/tables/policy_map.h:24 (kConvPolicyMap).
#pragma once

#include <cstdint>
#include <vector>

namespace lc0mi {

// 64*64 from->to entries followed by 8*24 promotion entries; -1 = no such move.
const std::vector<int16_t>& AttnPolicyMap();
// 73 planes x 64 squares; -1 = no such move.
const std::vector<int16_t>& ConvPolicyMap();
// 64 x 64 floats: -1 on the diagonal, 1 where a queen or knight move exists.
const std::vector<float>& PosEncoding();
// For each of the 1858 policy outputs, its source index in the attention map.
const std::vector<int16_t>& AttnPolicyInverseMap();
// For each of the 1858 policy outputs, its source index in the conv map.
const std::vector<int16_t>& ConvPolicyInverseMap();

}  // namespace lc0mi
