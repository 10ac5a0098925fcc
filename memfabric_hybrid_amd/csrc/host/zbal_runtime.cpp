/*
 * Library-level entry points: version, logger, last error, bootstrap
 * (reference zbal.cpp, zbal_bootstrap.cpp, common/zbal_logger.h,
 * common/zbal_last_error.h). The bootstrap is the single-process case: it
 * binds the HIP device and records the world shape; there is no rendezvous
 * and no symmetric heap, peers being windows registered per communicator.
 */
#include <atomic>
#include <cerrno>
#include <csignal>
#include <cstdio>
#include <cstring>
#include <thread>

#include <semaphore.h>

#include <hip/hip_runtime.h>

#include "zbal_host.h"

#ifndef ZBAL_VERSION_STRING
#define ZBAL_VERSION_STRING "zbal-mi355x 0.1.0 (gfx950)"
#endif

namespace zbal {

namespace {
std::atomic<int> gLogLevel{LOG_WARN};
std::atomic<void (*)(int, const char *)> gLogSink{nullptr};
thread_local std::string tLastError;
thread_local std::string tLastErrorReturned;
std::mutex gBootMutex;
} // namespace

bool LogEnabled(int level) { return level >= gLogLevel.load(std::memory_order_relaxed); }

void LogWrite(int level, const std::string &text)
{
    if (!LogEnabled(level)) return;
    auto sink = gLogSink.load(std::memory_order_acquire);
    if (sink) {
        sink(level, text.c_str());
        return;
    }
    static const char *names[] = {"DEBUG", "INFO", "WARN", "ERROR"};
    std::fprintf(stderr, "[zbal][%s] %s\n", names[level < 0 ? 0 : (level > 3 ? 3 : level)], text.c_str());
}

void SetLastError(const std::string &text) { tLastError = text; }

BootState &Boot()
{
    static BootState state;
    return state;
}

} // namespace zbal

using namespace zbal;

/*
 * SIGUSR1 asks for every communicator's device trace, as in the reference (common/zbal_signal_handler.cpp:21-29).
 * Writing the traces takes the registry's lock, synchronises the device, allocates and writes files: nothing a
 * signal handler may do (the signal can land on a thread that holds that very lock). The handler only posts a
 * semaphore and passes the signal on to the handler that was installed before bootstrap; a helper thread, started by
 * bootstrap and joined by unbootstrap, waits on the semaphore and writes the traces from ordinary code -- also when
 * every other thread of the process is stuck, which is when one wants them.
 */
namespace {
sem_t gDumpRequests;
std::atomic<bool> gDumpThreadStop{false};
std::thread gDumpThread;
struct sigaction gPreviousUsr1;
bool gHandlerInstalled = false;

void OnUsr1(int sig, siginfo_t *info, void *context)
{
    const int saved = errno;
    sem_post(&gDumpRequests);
    errno = saved;
    if (gPreviousUsr1.sa_flags & SA_SIGINFO) {
        if (gPreviousUsr1.sa_sigaction != nullptr) gPreviousUsr1.sa_sigaction(sig, info, context);
    } else if (gPreviousUsr1.sa_handler != SIG_DFL && gPreviousUsr1.sa_handler != SIG_IGN && gPreviousUsr1.sa_handler != nullptr) {
        gPreviousUsr1.sa_handler(sig);
    }
}

void DumpThreadMain()
{
    for (;;) {
        while (sem_wait(&gDumpRequests) != 0 && errno == EINTR) {}
        if (gDumpThreadStop.load(std::memory_order_acquire)) return;
        registry::DumpAllTraces();
    }
}

void InstallUsr1()
{
    sem_init(&gDumpRequests, 0, 0);
    gDumpThreadStop.store(false, std::memory_order_release);
    gDumpThread = std::thread(DumpThreadMain);
    struct sigaction act;
    std::memset(&act, 0, sizeof(act));
    act.sa_sigaction = OnUsr1;
    act.sa_flags = SA_SIGINFO | SA_RESTART;
    sigemptyset(&act.sa_mask);
    gHandlerInstalled = sigaction(SIGUSR1, &act, &gPreviousUsr1) == 0;
}

void RemoveUsr1()
{
    if (gHandlerInstalled) { /* the process gets back the SIGUSR1 handler it had before bootstrap */
        sigaction(SIGUSR1, &gPreviousUsr1, nullptr);
        gHandlerInstalled = false;
    }
    if (gDumpThread.joinable()) {
        gDumpThreadStop.store(true, std::memory_order_release);
        sem_post(&gDumpRequests);
        gDumpThread.join();
        sem_destroy(&gDumpRequests);
    }
}

/*
 * A process may end (or unload the library) without calling unbootstrap: the helper thread is then still waiting, and
 * a std::thread destroyed while joinable ends the process with std::terminate. This object is defined after the
 * thread, so it is destroyed first and takes the thread down the ordinary way.
 */
struct DumpThreadAtExit {
    ~DumpThreadAtExit() { RemoveUsr1(); }
} gDumpThreadAtExit;
} // namespace

/* the kernel launchers' way to leave a last-error text (declared in kernels/zbal_device.h) */
void zbalhip_set_last_error(const char *text) { ZBAL_LOG_AND_SET_LAST_ERROR(text); }

extern "C" {

__attribute__((visibility("default"))) const char *zbal_version() { return ZBAL_VERSION_STRING; }

__attribute__((visibility("default"))) int32_t zbal_set_logger(void (*func)(int, const char *))
{
    gLogSink.store(func, std::memory_order_release);
    return Z_OK;
}

__attribute__((visibility("default"))) int32_t zbal_set_logger_level(int level)
{
    if (level < LOG_DEBUG || level > LOG_ERROR) {
        SetLastError("logger level must be 0..3");
        return Z_INVALID_PARAM;
    }
    gLogLevel.store(level, std::memory_order_relaxed);
    return Z_OK;
}

__attribute__((visibility("default"))) const char *zbal_get_last_error_msg() { return tLastError.c_str(); }

__attribute__((visibility("default"))) const char *zbal_get_and_clear_last_error_msg()
{
    tLastErrorReturned.swap(tLastError);
    tLastError.clear();
    return tLastErrorReturned.c_str();
}

__attribute__((visibility("default"))) int32_t zbal_bootstrap_options_init(zbal_bootstrap_options_t *options)
{
    ZBAL_VALIDATE_RETURN(options != nullptr, "Init bootstrap options failed as options is null", Z_INVALID_PARAM);
    std::memset(options, 0, sizeof(*options));
    options->btType = BOOT_BY_MEMFABRIC;
    options->worldSize = 1;
    options->commMetaSpaceSize = 1024;
    options->commGroupCap = 128;
    return Z_OK;
}

__attribute__((visibility("default"))) int32_t zbal_bootstrap(zbal_bootstrap_options_t *options,
                                                              zbal_bootstrap_output_t *output)
{
    ZBAL_VALIDATE_RETURN(options != nullptr, "Bootstrap failed as options is null", Z_INVALID_PARAM);
    ZBAL_VALIDATE_RETURN(options->worldSize > 0, "Bootstrap failed as worldSize is 0", Z_INVALID_PARAM);
    ZBAL_VALIDATE_RETURN(options->rankId < options->worldSize,
                         "Bootstrap failed as rankId " << options->rankId << " is not below worldSize "
                                                       << options->worldSize,
                         Z_INVALID_PARAM);
    std::lock_guard<std::mutex> guard(gBootMutex);
    BootState &st = Boot();
    ZBAL_VALIDATE_RETURN(!st.bootstrapped, "Bootstrap failed as already bootstrapped", Z_INIT_BOOTSTRAP_FAILED);
    /* flags bit 0: host-only bootstrap (no device is touched); used with the do-nothing backend */
    if ((options->flags & 1u) == 0) {
        int ndev = 0;
        hipError_t e = hipGetDeviceCount(&ndev);
        ZBAL_VALIDATE_RETURN(e == hipSuccess && ndev > 0, "Bootstrap failed as no HIP device is visible",
                             Z_INIT_BOOTSTRAP_FAILED);
        ZBAL_VALIDATE_RETURN(options->deviceId < ndev, "Bootstrap failed as deviceId " << options->deviceId
                                                                                       << " is out of range",
                             Z_INVALID_PARAM);
        e = hipSetDevice(options->deviceId);
        ZBAL_VALIDATE_RETURN(e == hipSuccess, "Bootstrap failed as hipSetDevice failed: " << hipGetErrorString(e),
                             Z_INIT_BOOTSTRAP_FAILED);
    }
    InstallUsr1(); /* installed by bootstrap, reference bootstrap/zbal_bootstrap_default.cpp:102 */
    st.bootstrapped = true;
    st.worldSize = options->worldSize;
    st.rankId = options->rankId;
    st.deviceId = options->deviceId;
    st.deviceMemorySize = options->deviceMemorySize;
    if (output) {
        std::memset(output, 0, sizeof(*output));
        output->createdDeviceMemorySpaceSize = options->deviceMemorySize * options->worldSize;
        output->allocatedDeviceMemorySize = 0; /* windows are supplied by the caller */
    }
    ZBAL_LOG(LOG_INFO, "bootstrapped: world " << st.worldSize << ", rank " << st.rankId << ", device " << st.deviceId);
    return Z_OK;
}

__attribute__((visibility("default"))) int32_t zbal_unbootstrap(uint32_t flags)
{
    (void)flags;
    std::lock_guard<std::mutex> guard(gBootMutex);
    BootState &st = Boot();
    ZBAL_VALIDATE_RETURN(st.bootstrapped, "Unbootstrap failed as not bootstrapped", Z_CANNOT_UNBOOTSTRAP);
    RemoveUsr1(); /* before the communicators go: the helper thread must not be writing their traces */
    registry::DestroyAll();
    st = BootState();
    return Z_OK;
}

} // extern "C"
