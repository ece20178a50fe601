// Only for the ThreadSanitizer builds (make tsan).  GCC 11's ThreadSanitizer
// runtime does not intercept pthread_cond_clockwait, which libstdc++'s
// condition_variable::wait_for uses: it then never learns that the wait gave
// the mutex up and reports a double lock the next time the mutex is taken.
// This definition, which the dynamic linker prefers to the C library's,
// forwards to pthread_cond_timedwait (which the runtime does know) with the
// deadline moved to the realtime clock.
#include <pthread.h>
#include <time.h>

extern "C" int pthread_cond_clockwait(pthread_cond_t *cond, pthread_mutex_t *mutex, clockid_t clock,
                                      const struct timespec *deadline)
{
    struct timespec here, real;
    clock_gettime(clock, &here);
    clock_gettime(CLOCK_REALTIME, &real);
    long long ns = (deadline->tv_sec - here.tv_sec) * 1000000000ll + (deadline->tv_nsec - here.tv_nsec);
    if (ns < 0) ns = 0;
    ns += real.tv_sec * 1000000000ll + real.tv_nsec;
    struct timespec target;
    target.tv_sec = (time_t)(ns / 1000000000ll);
    target.tv_nsec = (long)(ns % 1000000000ll);
    return pthread_cond_timedwait(cond, mutex, &target);
}
