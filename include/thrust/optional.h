// Named by the API this front end mirrors and not provided by it.  The header exists so that
// including it stops the build here, instead of the compiler picking up a file of the same name
// from another Thrust installation on its include path and mixing two implementations.
#pragma once
#error "thrust::optional is not provided by this Thrust front end (MI355X device system: the sort / scan / reduce / select / merge path and its callers)"
