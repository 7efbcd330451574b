// Host stand-in for <hip/hip_bf16.h>: the library only uses the compiler's own __bf16 type.
#pragma once
