// Named by the API this front end mirrors and not provided by it.  The header exists so that
// including it stops the build here, instead of the compiler picking up a file of the same name
// from another Thrust installation on its include path and mixing two implementations.
#pragma once
#error "this Thrust front end does not provide the CUDA system (the device system here is thrust::hip, see thrust/execution_policy.h)"
