// Attention kernel variants for head dim 128.
#include "attention_dispatch.hpp"
namespace risa {
RISA_DEFINE_ATTENTION_VARIANT(128)
}  // namespace risa
