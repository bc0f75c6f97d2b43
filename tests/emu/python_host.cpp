// Test infrastructure: the Python interpreter as a program that carries the ThreadSanitizer runtime, so that the
// race-checked CPU build of the kernels (a shared library whose sanitizer calls the loading program has to provide) can
// be loaded by the same pytest files that drive the plain CPU build.  Python and its extension modules are not
// instrumented: the sanitizer sees the kernels' accesses and the threads that stand for wavefronts, nothing else.
#include <Python.h>

int main(int argc, char **argv) { return Py_BytesMain(argc, argv); }
