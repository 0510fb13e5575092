// Error plumbing shared by the host sources.
#pragma once
#include <cstdarg>
#include <cstdint>
#include <string>

#include "../../../include/cutile_hip.h"
#include "hip_api.h"

namespace cutile {

// Records `status` with a printf-style message for the calling thread and
// returns `status`, so call sites can `return fail(...)`.
cutile_status_t fail(cutile_status_t status, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
// Maps a hipError_t to a status (hipSuccess -> 0), recording the runtime's message.
cutile_status_t from_hip(hipError_t err, const char* what);
void clear_error();

#define CUTILE_HIP_OR_RETURN(api, call)                         \
  do {                                                          \
    hipError_t _e = (api)->call;                                \
    if (_e != hipSuccess) return ::cutile::from_hip(_e, #call); \
  } while (0)

#define CUTILE_API_OR_RETURN(api)                                  \
  const ::cutile::HipApi* api = ::cutile::hip();                   \
  if (!api) return CUTILE_ERR_LIBRARY_INIT

#define CUTILE_REQUIRE(cond, status, ...) \
  do {                                    \
    if (!(cond)) return ::cutile::fail(status, __VA_ARGS__); \
  } while (0)

}  // namespace cutile
