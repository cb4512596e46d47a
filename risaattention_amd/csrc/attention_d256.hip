// Attention kernel variants for head dim 256.
#include "attention_dispatch.hpp"
namespace risa {
RISA_DEFINE_ATTENTION_VARIANT(256)
}  // namespace risa
