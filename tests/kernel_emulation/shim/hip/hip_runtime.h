// Stand-in for <hip/hip_runtime.h> when a kernel header is compiled for the host by tests/test_kernel_emulation.py:
// the qualifiers vanish, threadIdx / blockIdx come from the fibre scheduler of emu.h, and the few AMDGPU builtins the
// kernels use become calls into it. TEST INFRASTRUCTURE ONLY.
#pragma once
#include "../../emu.h"
