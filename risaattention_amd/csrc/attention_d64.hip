// Attention kernel variants for head dim 64.
#include "attention_dispatch.hpp"
namespace risa {
RISA_DEFINE_ATTENTION_VARIANT(64)
}  // namespace risa
