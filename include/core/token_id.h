// Token id type of the embedding and loss operators (reference: bpe::TokenId, 32-bit unsigned).
#pragma once

#include <cstdint>

namespace bpe {
using TokenId = std::uint32_t;
}
