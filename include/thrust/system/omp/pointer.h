// <thrust/system/omp/pointer.h> is a header of the Thrust API that the cdna4 device system does not provide.
// The file exists so that including it stops here with a clear message instead of resolving to
// another Thrust installation further down the include path and mixing two libraries.
#error "<thrust/system/omp/pointer.h> is not provided by the cdna4 device system"
