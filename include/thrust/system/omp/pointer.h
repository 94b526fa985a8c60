// Named by the API this front end mirrors and not provided by it.  The header exists so that
// including it stops the build here, instead of the compiler picking up a file of the same name
// from another Thrust installation on its include path and mixing two implementations.
#pragma once
#error "this Thrust front end does not provide the OpenMP system (the host system here is the sequential one, thrust::cpp)"
