/* libllc_entry.so: the symbol the reference's loader resolves.  Execution::load looks up `main` in the
 * compiled library and calls it as void(void**) (src/Compiler/Execution.cpp:12-16,
 * include/llcompiler/Compiler/Execution.h:23); this forwards to the plan bound in libllc_hip.so. */
#include "llc_hip.h"

void main(void** params) { llc_hip_entry(params); }
