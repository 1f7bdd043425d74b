/* Name shim: EmitC-generated host code includes "MTRTRuntimeStatus.h"
 * (mlir-tensorrt/compiler/lib/Passes/2_Host/HostToEmitC/EmitCppSupportFiles.cpp:209-213).  With
 * -I<this directory> on the compile line that include resolves here and pulls in the HIP flavour of the
 * StandaloneCPP runtime, so the generated file compiles unchanged. */
#include "../mtrt_hip_standalone.h"
