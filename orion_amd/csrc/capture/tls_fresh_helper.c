/* liborion_tlsfresh.so: one thread-local variable and a function that touches
 * it.  libinttemp.so loads a fresh copy of this library after other libraries
 * have been loaded or unloaded and has its client threads call the function:
 * on glibc before 2.39 that brings a thread's table of thread-local blocks up
 * to date and takes every later thread-local access of the thread -- the
 * framework's own included -- off the dynamic loader's slow path
 * (capture/tls_fresh.h has the whole story). */
static __thread unsigned long touched;

unsigned long orion_tls_touch(void) { return ++touched; }
