// Translation unit of the stand-alone gfx950 code object: every kernel entry
// point of blit_kernels.h and nothing else.  Compiled device-only into an ELF
// that the AQL path loads with hsa_executable_load_agent_code_object, the
// counterpart of the per-target shader blobs the reference generates from
// blit_shaders/*.s (projects/rocr-runtime/runtime/hsa-runtime/core/runtime/
// blit_shaders/CMakeLists.txt:52-166).
#include "blit_kernels.h"
