// The library's error text lives in runtime.hip, which a host-only sanitizer build leaves out.
#include <cstdarg>
namespace shrike { void set_error(const char *, ...) {} }
