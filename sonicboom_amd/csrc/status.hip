// The error slot and the build description of the kernel library.
#include "common.h"

namespace sb {
char *error_slot() {
  static thread_local char slot[kErrorLen] = {0};
  return slot;
}
}  // namespace sb

#ifndef SB_BUILD_FLAGS
#define SB_BUILD_FLAGS ""
#endif

#define SB_STR_(x) #x
#define SB_STR(x) SB_STR_(x)

extern "C" const char *sb_last_error(void) { return sb::error_slot(); }

extern "C" const char *sb_build_info(void) {
  return "{\"library\": \"sonicboom_amd\", \"target\": \"gfx950\", \"wave\": 64, "
         "\"page\": " SB_STR(SB_PAGE) ", \"flags\": \"" SB_BUILD_FLAGS "\"}";
}
