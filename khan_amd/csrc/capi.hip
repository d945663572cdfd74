// extern "C" surface of libkhan_aev.so: argument checks and dispatch to the kernel launchers.
#include <atomic>
#include <cstdlib>
#include <mutex>
#include <string>

#include "../../include/khan_aev.h"
#include "khan_internal.h"
#include "khan_params.h"

// Size order of khan_featurize_f32_noalloc: the molecule indices by decreasing atom count, then the class counts
// and cursors (khan::launch_size_order).  One copy per GPU, held until the process ends.  In host code this name
// is a stand-in, not a device address: host code uses the pointer that noalloc_scratch() returns.
static __device__ __align__(256) int32_t scratch[KHAN_FEATURIZE_NOALLOC_MAX_MOLS + khan::kSizeOrderScratch];

namespace {

thread_local std::string g_last_hip_error;

// khan_set_reproducible_gradients: the one setting of the library (process-wide, read at every gradient call)
std::atomic<int> g_reproducible{0};

// Device address of `scratch` on the current device, looked up once per device with that device current.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
int32_t* g_scratch_ptr[kMaxDevices] = {};

hipError_t noalloc_scratch(int32_t** ptr)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (!p) return hipErrorInvalidSymbol;
        g_scratch_ptr[dev] = static_cast<int32_t*>(p);
    }
    *ptr = g_scratch_ptr[dev];
    return hipSuccess;
}

int hip_status(hipError_t e)
{
    if (e == hipSuccess) return KHAN_OK;
    g_last_hip_error = hipGetErrorString(e);
    return KHAN_ERR_HIP;
}

inline hipStream_t as_stream(khan_stream_t s) { return static_cast<hipStream_t>(s); }

// Check build only (-DKHAN_CHECK_BUILD, khan_amd/build.py: build_check_variant): KHAN_AEV_FORCE_GENERIC=1 in the
// environment routes every molecule through the general-shape kernels, KHAN_AEV_LARGE_SCRATCH=0 withholds the large
// molecules' scratch (both read once), so that tests reach those paths on ordinary inputs.  The default library
// reads no environment variable here.
#ifdef KHAN_CHECK_BUILD
bool force_generic()
{
    static const bool v = [] {
        const char* e = getenv("KHAN_AEV_FORCE_GENERIC");
        return e && e[0] == '1';
    }();
    return v;
}
bool large_scratch_withheld()
{
    static const bool v = [] {
        const char* e = getenv("KHAN_AEV_LARGE_SCRATCH");
        return e && e[0] == '0';
    }();
    return v;
}
#else
constexpr bool force_generic() { return false; }
constexpr bool large_scratch_withheld() { return false; }
#endif

// below a few thousand molecules every wavefront of a launch is resident at once and the size order buys nothing
constexpr int32_t kSizeOrderMinMols = 2048;

template <typename T>
bool aligned16(const khan::Buckets<const T>& g)
{
    for (int t = 0; t < 4; ++t)
        if (reinterpret_cast<uintptr_t>(g.p[t]) & 15u) return false;
    return true;
}

// Stream-ordered scratch holding the molecule indices by decreasing size for the one-wavefront kernels.
// No order (the kernels then take molecules as they come) while the stream is being captured into a graph,
// for small batches, or when the allocation fails.
class SizeOrder {
public:
    SizeOrder(const int32_t* macs, int32_t n_mols, hipStream_t stream) : stream_(stream)
    {
        if (n_mols < kSizeOrderMinMols) return;
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) {
            (void)hipGetLastError();
            return;
        }
        if (hipMallocAsync(reinterpret_cast<void**>(&order_), sizeof(int32_t) * (static_cast<size_t>(n_mols) + khan::kSizeOrderScratch), stream) != hipSuccess) {
            (void)hipGetLastError();
            order_ = nullptr;
            return;
        }
        if (khan::launch_size_order(macs, n_mols, order_, stream) != hipSuccess) {
            (void)hipGetLastError();
            (void)hipFreeAsync(order_, stream);
            order_ = nullptr;
        }
    }
    ~SizeOrder()
    {
        if (order_) (void)hipFreeAsync(order_, stream_);
    }
    SizeOrder(const SizeOrder&) = delete;
    SizeOrder& operator=(const SizeOrder&) = delete;
    const int32_t* get() const { return order_; }

private:
    int32_t* order_ = nullptr;
    hipStream_t stream_;
};

// Stream-ordered scratch for the type-sorted copy of the molecules of more than 256 atoms.  None while the stream is
// being captured into a graph, when the caller may not allocate, or when the allocation fails: those molecules then
// go through the general-shape kernels, which need no scratch.
class LargeScratch {
public:
    LargeScratch(size_t bytes, hipStream_t stream) : stream_(stream)
    {
        if (bytes == 0 || large_scratch_withheld()) return;
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) {
            (void)hipGetLastError();
            return;
        }
        if (hipMallocAsync(&p_, bytes, stream) != hipSuccess) {
            (void)hipGetLastError();
            p_ = nullptr;
        }
    }
    ~LargeScratch()
    {
        if (p_) (void)hipFreeAsync(p_, stream_);
    }
    LargeScratch(const LargeScratch&) = delete;
    LargeScratch& operator=(const LargeScratch&) = delete;
    void* get() const { return p_; }

private:
    void* p_ = nullptr;
    hipStream_t stream_;
};

// (the kernels for large molecules keep an atom's position inside its molecule in 28 bits)
constexpr int64_t kLargeAtomLimit = int64_t(1) << 28;

// Which kernels have work.  `classes` (host memory, null = not known: launch everything) holds the number of molecules
// of up to 32 atoms, of 33..64, of 65..256 and of more, as khan_size_order leaves them behind the order.
struct SizeClasses {
    bool known;
    int32_t n[khan::kSizeClasses];
    explicit SizeClasses(const int32_t* host) : known(host != nullptr)
    {
        for (int c = 0; c < khan::kSizeClasses; ++c) n[c] = host ? host[c] : 1;
    }
    // any molecule with lo <= atom count <= hi (lo, hi on class boundaries)?
    bool any(int lo, int hi) const
    {
        if (!known) return true;
        static const int first[khan::kSizeClasses] = {0, 33, 65, 257};
        for (int c = 0; c < khan::kSizeClasses; ++c) {
            const int last = c + 1 < khan::kSizeClasses ? first[c + 1] - 1 : INT32_MAX;
            if (first[c] >= lo && last <= hi && n[c] > 0) return true;
        }
        return false;
    }
};

// forward: one wavefront per molecule up to 32 atoms (float32; 64 in float64), one workgroup up to 256, several
// workgroups above (on a sorted copy of the atoms in scratch memory; without scratch, the general kernel)
template <typename T>
int forward_dispatch(const T* xs, const T* ys, const T* zs, const int32_t* as, const int32_t* mos,
                     const int32_t* macs, int32_t n_mols, const int32_t* sis, khan::Buckets<T> out,
                     const int32_t* order, const int32_t* classes_host, int64_t n_atoms, bool may_allocate,
                     hipStream_t stream)
{
    if (force_generic())
        return hip_status(khan::launch_fwd_generic<T>(xs, ys, zs, as, mos, macs, n_mols, sis, out, 0, nullptr, stream));
    constexpr int small_max = sizeof(T) == 4 ? khan::kSmallPreferredMax : khan::kSmallMaxAtoms;
    const SizeClasses cls(classes_host);
    int st = KHAN_OK;
    if (cls.any(0, small_max))
        st = hip_status(khan::launch_fwd_small<T>(xs, ys, zs, as, mos, macs, n_mols, sis, out, small_max, order, stream));
    if (st == KHAN_OK && cls.any(small_max + 1, khan::kMediumMaxAtoms))
        st = hip_status(khan::launch_fwd_medium<T>(xs, ys, zs, as, mos, macs, n_mols, sis, out, small_max + 1, order, stream));
    if (st == KHAN_OK && n_atoms > khan::kMediumMaxAtoms && cls.any(khan::kMediumMaxAtoms + 1, INT32_MAX)) {      // (n_atoms: of the whole batch)
        const LargeScratch scratch(may_allocate && n_atoms < kLargeAtomLimit ? khan::large_scratch_bytes<T>(n_atoms, n_mols, false) : 0, stream);
        if (scratch.get())
            st = hip_status(khan::launch_fwd_large<T>(xs, ys, zs, as, mos, macs, n_mols, sis, nullptr, nullptr, nullptr, out,
                                                      order, scratch.get(), n_atoms, stream));
        else
            st = hip_status(khan::launch_fwd_generic<T>(xs, ys, zs, as, mos, macs, n_mols, sis, out,
                                                        khan::kMediumMaxAtoms + 1, order, stream));
    }
    return st;
}

// backward: the same split; each kernel defines every gradient of its own molecules
template <typename T>
int backward_dispatch(const T* xs, const T* ys, const T* zs, const int32_t* as, const int32_t* mos,
                      const int32_t* macs, int32_t n_mols, const int32_t* sis, khan::Buckets<const T> g,
                      T* gx, T* gy, T* gz, int64_t n_atoms, const int32_t* order, const int32_t* classes_host,
                      hipStream_t stream)
{
    // the specialised kernels fetch upstream rows in 16-byte pieces; buckets that are not 16-byte aligned
    // (rows are 1,536 bytes, so the bucket's base decides) go through the general kernel, which does not care
    if (force_generic() || !aligned16(g))
        return hip_status(khan::launch_bwd_generic<T>(xs, ys, zs, as, mos, macs, n_mols, sis, g, gx, gy, gz,
                                                      n_atoms, 0, nullptr, stream));
    constexpr int small_max = sizeof(T) == 4 ? khan::kSmallPreferredMax : khan::kSmallMaxAtoms;
    const SizeClasses cls(classes_host);
    int st = KHAN_OK;
    if (n_atoms > khan::kMediumMaxAtoms && cls.any(khan::kMediumMaxAtoms + 1, INT32_MAX)) {
        const LargeScratch scratch(n_atoms < kLargeAtomLimit ? khan::large_scratch_bytes<T>(n_atoms, n_mols, false) : 0, stream);
        if (scratch.get())
            st = hip_status(khan::launch_bwd_large<T>(xs, ys, zs, as, mos, macs, n_mols, sis, g, gx, gy, gz, order,
                                                      scratch.get(), n_atoms, stream));
        else
            st = hip_status(khan::launch_bwd_generic<T>(xs, ys, zs, as, mos, macs, n_mols, sis, g, gx, gy, gz,
                                                        n_atoms, khan::kMediumMaxAtoms + 1, order, stream));
    }
    // The workgroup-per-molecule kernel walks the molecules in order of decreasing size: a launch lasts only a few
    // molecules' time (4,096 boxes on 1,024 workgroup slots), and in batch order it ended on whatever the batch had
    // last -- a quarter of the wavefront slots stood empty on average (boxes4096: 0.90 -> 0.73 ms)
    if (st == KHAN_OK && cls.any(small_max + 1, khan::kMediumMaxAtoms))
        st = hip_status(khan::launch_bwd_medium<T>(xs, ys, zs, as, mos, macs, n_mols, sis, g, gx, gy, gz,
                                                   small_max + 1, order, true, g_reproducible.load(std::memory_order_relaxed) != 0, stream));
    if (st == KHAN_OK && cls.any(0, small_max))
        st = hip_status(khan::launch_bwd_small<T>(xs, ys, zs, as, mos, macs, n_mols, sis, g, gx, gy, gz,
                                                  small_max, order, stream));
    return st;
}

// zeros to the four buckets (a batch with atoms but no molecule: the reference zero-fills its outputs before it
// looks at the molecules, functor_op_cpu.cpp:31-38)
template <typename T>
int zero_buckets(T* h, T* c, T* n, T* o, const int32_t* acs_host, hipStream_t stream)
{
    T* p[4] = {h, c, n, o};
    for (int t = 0; t < 4; ++t) {
        if (acs_host[t] > 0 && !p[t]) return KHAN_ERR_INVALID_ARG;
        const int st = hip_status(khan::launch_zero<T>(p[t], static_cast<int64_t>(acs_host[t]) * khan::kFeats, stream));
        if (st != KHAN_OK) return st;
    }
    return KHAN_OK;
}

// Argument checks of featurize and featurize_grad_inverse, and the batches that need no AEV kernel: KHAN_OK with
// *run == false means the call is complete (nothing to do, or rows of zeros written for atoms without a molecule).
template <typename T>
int featurize_check(const T* xs, const T* ys, const T* zs, const int32_t* as, const int32_t* mos,
                    const int32_t* macs, int32_t n_mols, const int32_t* sis, T* h, T* c, T* n, T* o,
                    const int32_t* acs_host, hipStream_t stream, bool* run)
{
    *run = false;
    if (n_mols < 0 || !acs_host) return KHAN_ERR_INVALID_ARG;
    if (acs_host[0] < 0 || acs_host[1] < 0 || acs_host[2] < 0 || acs_host[3] < 0) return KHAN_ERR_INVALID_ARG;
    const int64_t n_atoms = static_cast<int64_t>(acs_host[0]) + acs_host[1] + acs_host[2] + acs_host[3];
    if (n_atoms == 0) return KHAN_OK;
    if (n_atoms > INT32_MAX) return KHAN_ERR_TOO_LARGE;
    if (n_mols == 0) return zero_buckets(h, c, n, o, acs_host, stream);
    if (!xs || !ys || !zs || !as || !mos || !macs || !sis) return KHAN_ERR_INVALID_ARG;
    if ((acs_host[0] && !h) || (acs_host[1] && !c) || (acs_host[2] && !n) || (acs_host[3] && !o))
        return KHAN_ERR_INVALID_ARG;
    *run = true;
    return KHAN_OK;
}

template <typename T>
int featurize_impl(const T* xs, const T* ys, const T* zs, const int32_t* as, const int32_t* mos,
                   const int32_t* macs, int32_t n_mols, const int32_t* sis, T* h, T* c, T* n, T* o,
                   const int32_t* acs_host, khan_stream_t stream, const int32_t* caller_order = nullptr,
                   const int32_t* classes_host = nullptr, bool own_order = true)
{
    bool run;
    const int st = featurize_check(xs, ys, zs, as, mos, macs, n_mols, sis, h, c, n, o, acs_host, as_stream(stream), &run);
    if (st != KHAN_OK || !run) return st;
    khan::Buckets<T> out{{h, c, n, o}};
    const int64_t n_atoms = static_cast<int64_t>(acs_host[0]) + acs_host[1] + acs_host[2] + acs_host[3];
    if (!own_order)       // the caller's size order (or none)
        return forward_dispatch<T>(xs, ys, zs, as, mos, macs, n_mols, sis, out, caller_order, classes_host, n_atoms, true,
                                   as_stream(stream));
    SizeOrder order(macs, n_mols, as_stream(stream));
    return forward_dispatch<T>(xs, ys, zs, as, mos, macs, n_mols, sis, out, order.get(), nullptr, n_atoms, true, as_stream(stream));
}

template <typename T>
int featurize_grad_impl(const T* xs, const T* ys, const T* zs, const int32_t* as, const int32_t* mos,
                        const int32_t* macs, int32_t n_mols, const int32_t* sis, const T* gh,
                        const T* gc, const T* gn, const T* go, T* gx, T* gy, T* gz,
                        const int32_t* acs_host, khan_stream_t stream, const int32_t* caller_order = nullptr,
                        const int32_t* classes_host = nullptr, bool own_order = true)
{
    if (n_mols < 0 || !acs_host) return KHAN_ERR_INVALID_ARG;
    if (acs_host[0] < 0 || acs_host[1] < 0 || acs_host[2] < 0 || acs_host[3] < 0) return KHAN_ERR_INVALID_ARG;
    const int64_t n_atoms = static_cast<int64_t>(acs_host[0]) + acs_host[1] + acs_host[2] + acs_host[3];
    if (n_atoms == 0) return KHAN_OK;
    if (n_atoms > INT32_MAX) return KHAN_ERR_TOO_LARGE;
    if (!gx || !gy || !gz) return KHAN_ERR_INVALID_ARG;
    // atoms but no molecules: nothing contributes; the reference zero-fills its outputs first (functor_op_cpu.cpp:68-72)
    if (n_mols == 0) {
        for (T* g : {gx, gy, gz}) {
            const int st = hip_status(khan::launch_zero<T>(g, n_atoms, as_stream(stream)));
            if (st != KHAN_OK) return st;
        }
        return KHAN_OK;
    }
    if (!xs || !ys || !zs || !as || !mos || !macs || !sis) return KHAN_ERR_INVALID_ARG;
    if ((acs_host[0] && !gh) || (acs_host[1] && !gc) || (acs_host[2] && !gn) || (acs_host[3] && !go))
        return KHAN_ERR_INVALID_ARG;
    khan::Buckets<const T> g{{gh, gc, gn, go}};
    if (!own_order)
        return backward_dispatch<T>(xs, ys, zs, as, mos, macs, n_mols, sis, g, gx, gy, gz, n_atoms, caller_order, classes_host,
                                    as_stream(stream));
    SizeOrder order(macs, n_mols, as_stream(stream));
    return backward_dispatch<T>(xs, ys, zs, as, mos, macs, n_mols, sis, g, gx, gy, gz, n_atoms, order.get(), nullptr, as_stream(stream));
}

template <typename T>
int featurize_grad_inverse_impl(const T* xs, const T* ys, const T* zs, const int32_t* as, const int32_t* mos,
                                const int32_t* macs, int32_t n_mols, const int32_t* sis, const T* vx,
                                const T* vy, const T* vz, T* h, T* c, T* n, T* o,
                                const int32_t* acs_host, khan_stream_t stream, const int32_t* caller_order = nullptr,
                                const int32_t* classes_host = nullptr, bool own_order = true)
{
    bool run;
    const int chk = featurize_check(xs, ys, zs, as, mos, macs, n_mols, sis, h, c, n, o, acs_host, as_stream(stream), &run);
    if (chk != KHAN_OK || !run) return chk;
    if (!vx || !vy || !vz) return KHAN_ERR_INVALID_ARG;
    khan::Buckets<T> out{{h, c, n, o}};
    if (force_generic())
        return hip_status(khan::launch_jvp_generic<T>(xs, ys, zs, as, mos, macs, n_mols, sis, vx, vy, vz, out, 0,
                                                      nullptr, as_stream(stream)));
    // molecules of up to 64 atoms: one wavefront each; 65..256: one workgroup each; the rest: general-shape kernel
    SizeOrder made(own_order ? macs : nullptr, own_order ? n_mols : 0, as_stream(stream));
    const int32_t* order = own_order ? made.get() : caller_order;
    const SizeClasses cls(own_order ? nullptr : classes_host);
    int st = KHAN_OK;
    if (cls.any(0, khan::kSmallMaxAtoms))
        st = hip_status(khan::launch_jvp_small<T>(xs, ys, zs, as, mos, macs, n_mols, sis, vx, vy, vz, out, order,
                                                  as_stream(stream)));
    if (st == KHAN_OK && cls.any(khan::kSmallMaxAtoms + 1, khan::kMediumMaxAtoms))
        st = hip_status(khan::launch_jvp_medium<T>(xs, ys, zs, as, mos, macs, n_mols, sis, vx, vy, vz, out,
                                                   khan::kSmallMaxAtoms + 1, order, as_stream(stream)));
    if (st == KHAN_OK && cls.any(khan::kMediumMaxAtoms + 1, INT32_MAX)) {
        const int64_t n_atoms = static_cast<int64_t>(acs_host[0]) + acs_host[1] + acs_host[2] + acs_host[3];
        const LargeScratch scratch(n_atoms > khan::kMediumMaxAtoms && n_atoms < kLargeAtomLimit ? khan::large_scratch_bytes<T>(n_atoms, n_mols, true) : 0,
                                   as_stream(stream));
        if (scratch.get())
            st = hip_status(khan::launch_fwd_large<T>(xs, ys, zs, as, mos, macs, n_mols, sis, vx, vy, vz, out, order,
                                                      scratch.get(), n_atoms, as_stream(stream)));
        else if (n_atoms > khan::kMediumMaxAtoms)
            st = hip_status(khan::launch_jvp_generic<T>(xs, ys, zs, as, mos, macs, n_mols, sis, vx, vy, vz, out,
                                                        khan::kMediumMaxAtoms + 1, order, as_stream(stream)));
    }
    return st;
}

template <typename T>
int charge_impl(const T* xs, const T* ys, const T* zs, const T* qs, const int32_t* mos,
                const int32_t* macs, int32_t n_mols, bool damped, T k, T* e, khan_stream_t stream)
{
    if (n_mols < 0) return KHAN_ERR_INVALID_ARG;
    if (n_mols == 0) return KHAN_OK;
    if (!xs || !ys || !zs || !qs || !mos || !macs || !e) return KHAN_ERR_INVALID_ARG;
    return hip_status(khan::launch_charge_energy<T>(xs, ys, zs, qs, mos, macs, n_mols, damped, k, e, as_stream(stream)));
}

template <typename T>
int charge_grad_impl(const T* xs, const T* ys, const T* zs, const T* qs, const int32_t* mos,
                     const int32_t* macs, int32_t n_mols, const T* grads, bool damped, T k, T* qg, T* gx, T* gy, T* gz,
                     bool want_xyz, khan_stream_t stream, T* energies = nullptr)
{
    if (n_mols < 0) return KHAN_ERR_INVALID_ARG;
    if (n_mols == 0) return KHAN_OK;
    if (!xs || !ys || !zs || !qs || !mos || !macs || !grads) return KHAN_ERR_INVALID_ARG;
    if (want_xyz ? (!gx || !gy || !gz) : !qg) return KHAN_ERR_INVALID_ARG;
    return hip_status(khan::launch_charge_grad<T>(xs, ys, zs, qs, mos, macs, n_mols, grads, damped, k, qg,
                                                  want_xyz ? gx : nullptr, gy, gz, energies, as_stream(stream)));
}

}  // namespace

// Per-molecule sums of the per-type network outputs, and the way back (khan_mol_energy_*).
template <typename T>
static int mol_energy_impl(const T* const* out_host4, const int32_t* as, const int32_t* sis, const int32_t* mos,
                           const int32_t* macs, int32_t n_mols, T* e, khan_stream_t stream)
{
    if (n_mols < 0) return KHAN_ERR_INVALID_ARG;
    if (n_mols == 0) return KHAN_OK;
    if (!out_host4 || !as || !sis || !mos || !macs || !e) return KHAN_ERR_INVALID_ARG;
    khan::Buckets<const T> in;
    for (int t = 0; t < 4; ++t) in.p[t] = out_host4[t];
    return hip_status(khan::launch_mol_sum<T>(in, as, sis, mos, macs, n_mols, e, as_stream(stream)));
}

template <typename T>
static int mol_energy_grad_impl(const T* e_grads, const int32_t* as, const int32_t* sis, const int32_t* mos,
                                const int32_t* macs, int32_t n_mols, T* const* grad_host4, khan_stream_t stream)
{
    if (n_mols < 0) return KHAN_ERR_INVALID_ARG;
    if (n_mols == 0) return KHAN_OK;
    if (!grad_host4 || !as || !sis || !mos || !macs || !e_grads) return KHAN_ERR_INVALID_ARG;
    khan::Buckets<T> out;
    for (int t = 0; t < 4; ++t) out.p[t] = grad_host4[t];
    return hip_status(khan::launch_mol_sum_grad<T>(e_grads, as, sis, mos, macs, n_mols, out, as_stream(stream)));
}


extern "C" {

int32_t khan_feature_size(void) { return khan::kFeats; }

int khan_size_order(const int32_t* macs, int32_t n_mols, int32_t* order, khan_stream_t stream)
{
    if (n_mols < 0) return KHAN_ERR_INVALID_ARG;
    if (!order) return KHAN_ERR_INVALID_ARG;
    if (n_mols > 0 && !macs) return KHAN_ERR_INVALID_ARG;
    return hip_status(khan::launch_size_order(macs, n_mols, order, as_stream(stream)));
}

const char* khan_status_string(int status)
{
    switch (status) {
        case KHAN_OK: return "ok";
        case KHAN_ERR_INVALID_ARG: return "invalid argument";
        case KHAN_ERR_HIP: return "HIP runtime error";
        case KHAN_ERR_TOO_LARGE: return "input too large for int32 indexing";
        default: return "unknown status";
    }
}

const char* khan_last_hip_error(void) { return g_last_hip_error.c_str(); }

void khan_get_parameters(float* r_rs, float* a_thetas, float* a_rs, float* scalars)
{
    static const float rrs[16] = {5.0000000e-01f, 7.5625000e-01f, 1.0125000e+00f, 1.2687500e+00f,
                                  1.5250000e+00f, 1.7812500e+00f, 2.0375000e+00f, 2.2937500e+00f,
                                  2.5500000e+00f, 2.8062500e+00f, 3.0625000e+00f, 3.3187500e+00f,
                                  3.5750000e+00f, 3.8312500e+00f, 4.0875000e+00f, 4.3437500e+00f};
    static const float ath[8] = {0.0000000e+00f, 7.8539816e-01f, 1.5707963e+00f, 2.3561945e+00f,
                                 3.1415927e+00f, 3.9269908e+00f, 4.7123890e+00f, 5.4977871e+00f};
    static const float ars[4] = {5.0000000e-01f, 1.1500000e+00f, 1.8000000e+00f, 2.4500000e+00f};
    for (int i = 0; i < 16; ++i) r_rs[i] = rrs[i];
    for (int i = 0; i < 8; ++i) a_thetas[i] = ath[i];
    for (int i = 0; i < 4; ++i) a_rs[i] = ars[i];
    scalars[0] = khan::kR_eta_f;
    scalars[1] = khan::kR_Rc_f;
    scalars[2] = khan::kA_Rc_f;
    scalars[3] = khan::kA_eta_f;
    scalars[4] = 8.0f;
    scalars[5] = khan::kChargeK_f;
}

int khan_mol_offsets(const int32_t* mol_idxs, int64_t n_atoms, int32_t n_mols, int32_t* macs,
                     int32_t* mos, khan_stream_t stream)
{
    if (n_atoms < 0 || n_mols < 0) return KHAN_ERR_INVALID_ARG;
    if (n_atoms > INT32_MAX) return KHAN_ERR_TOO_LARGE;
    if (n_mols == 0) return KHAN_OK;
    if (!macs || !mos || (n_atoms > 0 && !mol_idxs)) return KHAN_ERR_INVALID_ARG;
    return hip_status(khan::launch_mol_offsets(mol_idxs, n_atoms, n_mols, macs, mos, as_stream(stream)));
}

int khan_ani_sort(const int32_t* atomic_numbers, int64_t n_atoms, int32_t* scatter_idxs,
                  int32_t* gather_idxs, int32_t* atom_counts, khan_stream_t stream)
{
    if (n_atoms < 0 || !atom_counts) return KHAN_ERR_INVALID_ARG;
    if (n_atoms > INT32_MAX) return KHAN_ERR_TOO_LARGE;
    if (n_atoms > 0 && (!atomic_numbers || !scatter_idxs || !gather_idxs)) return KHAN_ERR_INVALID_ARG;
    return hip_status(khan::launch_ani_sort(atomic_numbers, n_atoms, scatter_idxs, gather_idxs, atom_counts,
                                            as_stream(stream)));
}

int khan_featurize_f32(const float* xs, const float* ys, const float* zs, const int32_t* as,
                       const int32_t* mos, const int32_t* macs, int32_t n_mols, const int32_t* sis,
                       float* h, float* c, float* n, float* o, const int32_t* acs_host,
                       khan_stream_t stream)
{
    return featurize_impl<float>(xs, ys, zs, as, mos, macs, n_mols, sis, h, c, n, o, acs_host, stream);
}
int khan_featurize_f64(const double* xs, const double* ys, const double* zs, const int32_t* as,
                       const int32_t* mos, const int32_t* macs, int32_t n_mols, const int32_t* sis,
                       double* h, double* c, double* n, double* o, const int32_t* acs_host,
                       khan_stream_t stream)
{
    return featurize_impl<double>(xs, ys, zs, as, mos, macs, n_mols, sis, h, c, n, o, acs_host, stream);
}

int khan_set_reproducible_gradients(int on)
{
    return g_reproducible.exchange(on ? 1 : 0, std::memory_order_relaxed);
}

// khan_featurize_f32 without any allocation: the size order goes to the file-scope array above.
int khan_featurize_f32_noalloc(const float* xs, const float* ys, const float* zs, const int32_t* as,
                               const int32_t* mos, const int32_t* macs, int32_t n_mols, const int32_t* sis,
                               float* h, float* c, float* n, float* o, const int32_t* acs_host,
                               khan_stream_t stream)
{
    bool run;
    const int st = featurize_check(xs, ys, zs, as, mos, macs, n_mols, sis, h, c, n, o, acs_host, as_stream(stream), &run);
    if (st != KHAN_OK || !run) return st;
    if (n_mols > KHAN_FEATURIZE_NOALLOC_MAX_MOLS) {
        g_last_hip_error = "khan_featurize_f32_noalloc: more molecules than its fixed scratch holds (KHAN_FEATURIZE_NOALLOC_MAX_MOLS)";
        return KHAN_ERR_TOO_LARGE;
    }
    int32_t* order = nullptr;
    hipError_t e = noalloc_scratch(&order);
    if (e != hipSuccess) return hip_status(e);
    if (n_mols < kSizeOrderMinMols) {
        order = nullptr;       // as khan_featurize_f32: every wavefront of so small a launch is resident at once
    } else {
        // the class counts and cursors behind the indices keep the last call's values: launch_size_order clears them
        // with a kernel first; the indices are all rewritten
        e = khan::launch_size_order(macs, n_mols, order, as_stream(stream));
        if (e != hipSuccess) return hip_status(e);
    }
    khan::Buckets<float> out{{h, c, n, o}};
    // (molecules of more than 256 atoms go through the general-shape kernels here: the faster ones need scratch memory)
    const int64_t n_atoms = static_cast<int64_t>(acs_host[0]) + acs_host[1] + acs_host[2] + acs_host[3];
    return forward_dispatch<float>(xs, ys, zs, as, mos, macs, n_mols, sis, out, order, nullptr, n_atoms, false, as_stream(stream));
}

int khan_featurize_grad_f32(const float* xs, const float* ys, const float* zs, const int32_t* as,
                            const int32_t* mos, const int32_t* macs, int32_t n_mols,
                            const int32_t* sis, const float* gh, const float* gc, const float* gn,
                            const float* go, float* gx, float* gy, float* gz,
                            const int32_t* acs_host, khan_stream_t stream)
{
    return featurize_grad_impl<float>(xs, ys, zs, as, mos, macs, n_mols, sis, gh, gc, gn, go, gx, gy, gz,
                                      acs_host, stream);
}
int khan_featurize_grad_f64(const double* xs, const double* ys, const double* zs, const int32_t* as,
                            const int32_t* mos, const int32_t* macs, int32_t n_mols,
                            const int32_t* sis, const double* gh, const double* gc, const double* gn,
                            const double* go, double* gx, double* gy, double* gz,
                            const int32_t* acs_host, khan_stream_t stream)
{
    return featurize_grad_impl<double>(xs, ys, zs, as, mos, macs, n_mols, sis, gh, gc, gn, go, gx, gy, gz,
                                       acs_host, stream);
}

int khan_featurize_grad_inverse_f32(const float* xs, const float* ys, const float* zs, const int32_t* as,
                                    const int32_t* mos, const int32_t* macs, int32_t n_mols,
                                    const int32_t* sis, const float* x_grads, const float* y_grads,
                                    const float* z_grads, float* h, float* c, float* n, float* o,
                                    const int32_t* acs_host, khan_stream_t stream)
{
    return featurize_grad_inverse_impl<float>(xs, ys, zs, as, mos, macs, n_mols, sis, x_grads, y_grads, z_grads,
                                              h, c, n, o, acs_host, stream);
}
int khan_featurize_grad_inverse_f64(const double* xs, const double* ys, const double* zs, const int32_t* as,
                                    const int32_t* mos, const int32_t* macs, int32_t n_mols,
                                    const int32_t* sis, const double* x_grads, const double* y_grads,
                                    const double* z_grads, double* h, double* c, double* n, double* o,
                                    const int32_t* acs_host, khan_stream_t stream)
{
    return featurize_grad_inverse_impl<double>(xs, ys, zs, as, mos, macs, n_mols, sis, x_grads, y_grads, z_grads,
                                               h, c, n, o, acs_host, stream);
}

int khan_ani_charge_f32(const float* xs, const float* ys, const float* zs, const float* qs,
                        const int32_t* mos, const int32_t* macs, int32_t n_mols, float* e,
                        khan_stream_t stream)
{
    return charge_impl<float>(xs, ys, zs, qs, mos, macs, n_mols, true, khan::kChargeK_f, e, stream);
}
int khan_ani_charge_f64(const double* xs, const double* ys, const double* zs, const double* qs,
                        const int32_t* mos, const int32_t* macs, int32_t n_mols, double* e,
                        khan_stream_t stream)
{
    return charge_impl<double>(xs, ys, zs, qs, mos, macs, n_mols, true, static_cast<double>(khan::kChargeK_f), e, stream);
}

int khan_ani_charge_grad_f32(const float* xs, const float* ys, const float* zs, const float* qs,
                             const int32_t* mos, const int32_t* macs, int32_t n_mols,
                             const float* grads, float* q_grads, khan_stream_t stream)
{
    return charge_grad_impl<float>(xs, ys, zs, qs, mos, macs, n_mols, grads, true, khan::kChargeK_f, q_grads, nullptr, nullptr,
                                   nullptr, false, stream);
}
int khan_ani_charge_grad_f64(const double* xs, const double* ys, const double* zs, const double* qs,
                             const int32_t* mos, const int32_t* macs, int32_t n_mols,
                             const double* grads, double* q_grads, khan_stream_t stream)
{
    return charge_grad_impl<double>(xs, ys, zs, qs, mos, macs, n_mols, grads, true, static_cast<double>(khan::kChargeK_f), q_grads, nullptr, nullptr,
                                    nullptr, false, stream);
}

int khan_ani_charge_grad_xyz_f32(const float* xs, const float* ys, const float* zs, const float* qs,
                                 const int32_t* mos, const int32_t* macs, int32_t n_mols,
                                 const float* grads, float* q_grads, float* gx, float* gy, float* gz,
                                 khan_stream_t stream)
{
    return charge_grad_impl<float>(xs, ys, zs, qs, mos, macs, n_mols, grads, true, khan::kChargeK_f, q_grads, gx, gy, gz, true, stream);
}
int khan_ani_charge_all_f32(const float* xs, const float* ys, const float* zs, const float* qs,
                            const int32_t* mos, const int32_t* macs, int32_t n_mols, const float* grads,
                            float* e, float* q_grads, float* gx, float* gy, float* gz, khan_stream_t stream)
{
    if (n_mols > 0 && !e) return KHAN_ERR_INVALID_ARG;
    return charge_grad_impl<float>(xs, ys, zs, qs, mos, macs, n_mols, grads, true, khan::kChargeK_f, q_grads, gx, gy, gz, true, stream, e);
}
int khan_ani_charge_all_f64(const double* xs, const double* ys, const double* zs, const double* qs,
                            const int32_t* mos, const int32_t* macs, int32_t n_mols, const double* grads,
                            double* e, double* q_grads, double* gx, double* gy, double* gz, khan_stream_t stream)
{
    if (n_mols > 0 && !e) return KHAN_ERR_INVALID_ARG;
    return charge_grad_impl<double>(xs, ys, zs, qs, mos, macs, n_mols, grads, true, static_cast<double>(khan::kChargeK_f), q_grads, gx, gy, gz, true, stream, e);
}
int khan_ani_charge_grad_xyz_f64(const double* xs, const double* ys, const double* zs,
                                 const double* qs, const int32_t* mos, const int32_t* macs,
                                 int32_t n_mols, const double* grads, double* q_grads, double* gx,
                                 double* gy, double* gz, khan_stream_t stream)
{
    return charge_grad_impl<double>(xs, ys, zs, qs, mos, macs, n_mols, grads, true, static_cast<double>(khan::kChargeK_f), q_grads, gx, gy, gz, true, stream);
}

int khan_dense_first_f32(const float* const* rows_host4, const int32_t* acs_host, const float* const* wt_host4,
                         const float* const* bias_host4, int32_t activation, float alpha, float* const* out_host4,
                         khan_stream_t stream)
{
    if (!rows_host4 || !acs_host || !wt_host4 || !bias_host4 || !out_host4) return KHAN_ERR_INVALID_ARG;
    if (activation != KHAN_ACT_NONE && activation != KHAN_ACT_CELU) return KHAN_ERR_INVALID_ARG;
    if (activation == KHAN_ACT_CELU && !(alpha > 0.0f)) return KHAN_ERR_INVALID_ARG;
    int64_t total = 0;
    for (int t = 0; t < 4; ++t) {
        if (acs_host[t] < 0) return KHAN_ERR_INVALID_ARG;
        if (acs_host[t] > 0 && (!rows_host4[t] || !wt_host4[t] || !bias_host4[t] || !out_host4[t])) return KHAN_ERR_INVALID_ARG;
        // 16-byte loads of rows and weights
        if (acs_host[t] > 0 && ((reinterpret_cast<uintptr_t>(rows_host4[t]) | reinterpret_cast<uintptr_t>(wt_host4[t])) & 15u))
            return KHAN_ERR_INVALID_ARG;
        total += acs_host[t];
    }
    if (total == 0) return KHAN_OK;
    if (total > INT32_MAX) return KHAN_ERR_TOO_LARGE;
    return hip_status(khan::launch_dense_first(rows_host4, acs_host, wt_host4, bias_host4, activation == KHAN_ACT_CELU, alpha,
                                               out_host4, as_stream(stream)));
}

int khan_dense_f32(const float* const* rows_host4, const int32_t* n_host4, int32_t k, int32_t n_out,
                   const float* const* wt_host4, const float* const* bias_host4, int32_t activation, float alpha,
                   const float* const* deriv_of_host4, float* const* out_host4, khan_stream_t stream)
{
    if (!rows_host4 || !n_host4 || !wt_host4 || !out_host4) return KHAN_ERR_INVALID_ARG;
    if (activation != KHAN_ACT_NONE && activation != KHAN_ACT_CELU) return KHAN_ERR_INVALID_ARG;
    if ((activation == KHAN_ACT_CELU || deriv_of_host4) && !(alpha > 0.0f)) return KHAN_ERR_INVALID_ARG;
    if (k <= 0 || k % 32 != 0 || n_out <= 0 || n_out % 64 != 0) return KHAN_ERR_INVALID_ARG;
    int64_t total = 0;
    for (int t = 0; t < 4; ++t) {
        if (n_host4[t] < 0) return KHAN_ERR_INVALID_ARG;
        if (n_host4[t] == 0) continue;
        if (!rows_host4[t] || !wt_host4[t] || !out_host4[t]) return KHAN_ERR_INVALID_ARG;
        if (bias_host4 && !bias_host4[t]) return KHAN_ERR_INVALID_ARG;
        if (deriv_of_host4 && !deriv_of_host4[t]) return KHAN_ERR_INVALID_ARG;
        // 16-byte loads of rows, activations and weights
        uintptr_t bits = reinterpret_cast<uintptr_t>(rows_host4[t]) | reinterpret_cast<uintptr_t>(wt_host4[t]);
        if (deriv_of_host4) bits |= reinterpret_cast<uintptr_t>(deriv_of_host4[t]);
        if (bits & 15u) return KHAN_ERR_INVALID_ARG;
        total += n_host4[t];
    }
    if (total == 0) return KHAN_OK;
    if (total > INT32_MAX) return KHAN_ERR_TOO_LARGE;
    return hip_status(khan::launch_dense(rows_host4, n_host4, k, n_out, wt_host4, bias_host4, activation == KHAN_ACT_CELU,
                                         alpha, deriv_of_host4, out_host4, as_stream(stream)));
}

int khan_dense_head_f32(const float* const* rows_host4, const int32_t* n_host4, int32_t k, int32_t n_out,
                        const float* const* wt_host4, const float* const* bias_host4, int32_t activation, float alpha,
                        const float* const* head_w_host4, const float* const* head_b_host4, float* const* out_host4,
                        float* const* head_out_host4, khan_stream_t stream)
{
    if (!rows_host4 || !n_host4 || !wt_host4 || !head_w_host4 || !out_host4 || !head_out_host4) return KHAN_ERR_INVALID_ARG;
    if (activation != KHAN_ACT_NONE && activation != KHAN_ACT_CELU) return KHAN_ERR_INVALID_ARG;
    if (activation == KHAN_ACT_CELU && !(alpha > 0.0f)) return KHAN_ERR_INVALID_ARG;
    if (k <= 0 || k % 32 != 0 || n_out != 64) return KHAN_ERR_INVALID_ARG;
    int64_t total = 0;
    for (int t = 0; t < 4; ++t) {
        if (n_host4[t] < 0) return KHAN_ERR_INVALID_ARG;
        if (n_host4[t] == 0) continue;
        if (!rows_host4[t] || !wt_host4[t] || !head_w_host4[t] || !out_host4[t] || !head_out_host4[t]) return KHAN_ERR_INVALID_ARG;
        if (bias_host4 && !bias_host4[t]) return KHAN_ERR_INVALID_ARG;
        if (head_b_host4 && !head_b_host4[t]) return KHAN_ERR_INVALID_ARG;
        if ((reinterpret_cast<uintptr_t>(rows_host4[t]) | reinterpret_cast<uintptr_t>(wt_host4[t])) & 15u) return KHAN_ERR_INVALID_ARG;
        total += n_host4[t];
    }
    if (total == 0) return KHAN_OK;
    if (total > INT32_MAX) return KHAN_ERR_TOO_LARGE;
    return hip_status(khan::launch_dense_head(rows_host4, n_host4, k, n_out, wt_host4, bias_host4, activation == KHAN_ACT_CELU,
                                              alpha, head_w_host4, head_b_host4, out_host4, head_out_host4, as_stream(stream)));
}

int khan_dense_head_grad_f32(const float* const* scale_host4, const float* const* head_w_host4, const int32_t* n_host4,
                             int32_t k, int32_t n_out, const float* const* wt_host4, float alpha,
                             const float* const* deriv_of_host4, float* const* out_host4, khan_stream_t stream)
{
    if (!scale_host4 || !head_w_host4 || !n_host4 || !wt_host4 || !deriv_of_host4 || !out_host4) return KHAN_ERR_INVALID_ARG;
    if (!(alpha > 0.0f)) return KHAN_ERR_INVALID_ARG;
    if (k <= 0 || k % 32 != 0 || n_out <= 0 || n_out % 64 != 0) return KHAN_ERR_INVALID_ARG;
    int64_t total = 0;
    for (int t = 0; t < 4; ++t) {
        if (n_host4[t] < 0) return KHAN_ERR_INVALID_ARG;
        if (n_host4[t] == 0) continue;
        if (!scale_host4[t] || !head_w_host4[t] || !wt_host4[t] || !deriv_of_host4[t] || !out_host4[t]) return KHAN_ERR_INVALID_ARG;
        // 16-byte loads of the output layer's weights, the activations and the weights
        if ((reinterpret_cast<uintptr_t>(head_w_host4[t]) | reinterpret_cast<uintptr_t>(wt_host4[t]) |
             reinterpret_cast<uintptr_t>(deriv_of_host4[t])) & 15u)
            return KHAN_ERR_INVALID_ARG;
        total += n_host4[t];
    }
    if (total == 0) return KHAN_OK;
    if (total > INT32_MAX) return KHAN_ERR_TOO_LARGE;
    return hip_status(khan::launch_dense_head_grad(scale_host4, head_w_host4, n_host4, k, n_out, wt_host4, alpha, deriv_of_host4,
                                                   out_host4, as_stream(stream)));
}

int64_t khan_atomic_networks_packed_bytes(void) { return static_cast<int64_t>(khan::networks_packed_bytes()); }

int khan_atomic_networks_pack_f32(const float* const* weights_t_host12, const float* const* weights_host12, void* packed,
                                  khan_stream_t stream)
{
    if (!weights_t_host12 || !weights_host12 || !packed) return KHAN_ERR_INVALID_ARG;
    for (int k = 0; k < 12; ++k)
        if (!weights_t_host12[k] || !weights_host12[k]) return KHAN_ERR_INVALID_ARG;
    if (reinterpret_cast<uintptr_t>(packed) & 15u) return KHAN_ERR_INVALID_ARG;
    return hip_status(khan::launch_networks_pack(weights_t_host12, weights_t_host12 + 4, weights_t_host12 + 8, weights_host12,
                                                 weights_host12 + 4, weights_host12 + 8, packed, as_stream(stream)));
}

int khan_atomic_networks_f32(const float* const* rows_host4, const int32_t* n_host4, const float* const* weights_t_host12,
                             const float* const* weights_host12, const void* packed, const float* const* biases_host12,
                             const float* const* head_w_host4, const float* const* head_b_host4,
                             const float* const* scale_host4, float alpha, float* const* value_host4,
                             float* const* grad_host4, khan_stream_t stream)
{
    if (!rows_host4 || !n_host4 || !biases_host12 || !head_w_host4 || !value_host4) return KHAN_ERR_INVALID_ARG;
    if (!packed && (!weights_t_host12 || (grad_host4 && !weights_host12))) return KHAN_ERR_INVALID_ARG;
    if (packed && (reinterpret_cast<uintptr_t>(packed) & 15u)) return KHAN_ERR_INVALID_ARG;
    if (!(alpha > 0.0f)) return KHAN_ERR_INVALID_ARG;
    int64_t total = 0;
    for (int t = 0; t < 4; ++t) {
        if (n_host4[t] < 0) return KHAN_ERR_INVALID_ARG;
        if (n_host4[t] == 0) continue;
        if (!rows_host4[t] || !head_w_host4[t] || !value_host4[t]) return KHAN_ERR_INVALID_ARG;
        uintptr_t bits = reinterpret_cast<uintptr_t>(rows_host4[t]);        // 16-byte loads of rows and weights
        for (int l = 0; l < 3; ++l) {
            if (!biases_host12[4 * l + t]) return KHAN_ERR_INVALID_ARG;
            if (packed) continue;
            if (!weights_t_host12[4 * l + t]) return KHAN_ERR_INVALID_ARG;
            bits |= reinterpret_cast<uintptr_t>(weights_t_host12[4 * l + t]);
            if (grad_host4) {
                if (!weights_host12[4 * l + t]) return KHAN_ERR_INVALID_ARG;
                bits |= reinterpret_cast<uintptr_t>(weights_host12[4 * l + t]);
            }
        }
        if (grad_host4 && !grad_host4[t]) return KHAN_ERR_INVALID_ARG;
        if (bits & 15u) return KHAN_ERR_INVALID_ARG;
        total += n_host4[t];
    }
    if (total == 0) return KHAN_OK;
    if (total > INT32_MAX) return KHAN_ERR_TOO_LARGE;
    const bool plain = !packed;
    return hip_status(khan::launch_networks_fused(
        rows_host4, n_host4, plain ? weights_t_host12 : nullptr, plain ? weights_t_host12 + 4 : nullptr,
        plain ? weights_t_host12 + 8 : nullptr, plain && weights_host12 ? weights_host12 : nullptr,
        plain && weights_host12 ? weights_host12 + 4 : nullptr, plain && weights_host12 ? weights_host12 + 8 : nullptr,
        biases_host12, biases_host12 + 4, biases_host12 + 8, head_w_host4, head_b_host4, scale_host4, alpha, value_host4,
        grad_host4, packed, as_stream(stream)));
}

// Per-molecule sums of the per-type network outputs, and the way back.
int khan_mol_energy_f32(const float* const* out_host4, const int32_t* as, const int32_t* sis, const int32_t* mos,
                        const int32_t* macs, int32_t n_mols, float* e, khan_stream_t stream)
{
    return mol_energy_impl<float>(out_host4, as, sis, mos, macs, n_mols, e, stream);
}
int khan_mol_energy_f64(const double* const* out_host4, const int32_t* as, const int32_t* sis, const int32_t* mos,
                        const int32_t* macs, int32_t n_mols, double* e, khan_stream_t stream)
{
    return mol_energy_impl<double>(out_host4, as, sis, mos, macs, n_mols, e, stream);
}
int khan_mol_energy_grad_f32(const float* e_grads, const int32_t* as, const int32_t* sis, const int32_t* mos,
                             const int32_t* macs, int32_t n_mols, float* const* grad_host4, khan_stream_t stream)
{
    return mol_energy_grad_impl<float>(e_grads, as, sis, mos, macs, n_mols, grad_host4, stream);
}
int khan_mol_energy_grad_f64(const double* e_grads, const int32_t* as, const int32_t* sis, const int32_t* mos,
                             const int32_t* macs, int32_t n_mols, double* const* grad_host4, khan_stream_t stream)
{
    return mol_energy_grad_impl<double>(e_grads, as, sis, mos, macs, n_mols, grad_host4, stream);
}

// Plain Coulomb sums: the charge kernels with the cutoff function switched off and the constant given by the caller.
int khan_coulomb_f32(const float* xs, const float* ys, const float* zs, const float* qs, const int32_t* mos,
                     const int32_t* macs, int32_t n_mols, float k, float* e, khan_stream_t stream)
{
    return charge_impl<float>(xs, ys, zs, qs, mos, macs, n_mols, false, k, e, stream);
}
int khan_coulomb_f64(const double* xs, const double* ys, const double* zs, const double* qs, const int32_t* mos,
                     const int32_t* macs, int32_t n_mols, double k, double* e, khan_stream_t stream)
{
    return charge_impl<double>(xs, ys, zs, qs, mos, macs, n_mols, false, k, e, stream);
}
int khan_coulomb_grad_f32(const float* xs, const float* ys, const float* zs, const float* qs, const int32_t* mos,
                          const int32_t* macs, int32_t n_mols, const float* grads, float k, float* q_grads,
                          float* gx, float* gy, float* gz, khan_stream_t stream)
{
    return charge_grad_impl<float>(xs, ys, zs, qs, mos, macs, n_mols, grads, false, k, q_grads, gx, gy, gz, true, stream);
}
int khan_coulomb_grad_f64(const double* xs, const double* ys, const double* zs, const double* qs, const int32_t* mos,
                          const int32_t* macs, int32_t n_mols, const double* grads, double k, double* q_grads,
                          double* gx, double* gy, double* gz, khan_stream_t stream)
{
    return charge_grad_impl<double>(xs, ys, zs, qs, mos, macs, n_mols, grads, false, k, q_grads, gx, gy, gz, true, stream);
}

// The AEV passes on a size order that the caller computed once for the batch (khan_size_order).  They allocate nothing,
// except for a batch that holds a molecule of more than 256 atoms: its sorted copy goes to stream-ordered scratch
// (with the class counts unknown on the host, for any batch of more than 256 atoms), unless the stream is being
// captured -- then those molecules take the general-shape kernels, which need none.
int khan_featurize_ordered_f32(const float* xs, const float* ys, const float* zs, const int32_t* as,
                               const int32_t* mos, const int32_t* macs, int32_t n_mols, const int32_t* sis,
                               float* h, float* c, float* n, float* o, const int32_t* acs_host,
                               const int32_t* order, const int32_t* size_classes_host,
        khan_stream_t stream)
{
    return featurize_impl<float>(xs, ys, zs, as, mos, macs, n_mols, sis, h, c, n, o, acs_host, stream, order, size_classes_host, false);
}
int khan_featurize_ordered_f64(const double* xs, const double* ys, const double* zs, const int32_t* as,
                               const int32_t* mos, const int32_t* macs, int32_t n_mols, const int32_t* sis,
                               double* h, double* c, double* n, double* o, const int32_t* acs_host,
                               const int32_t* order, const int32_t* size_classes_host,
        khan_stream_t stream)
{
    return featurize_impl<double>(xs, ys, zs, as, mos, macs, n_mols, sis, h, c, n, o, acs_host, stream, order, size_classes_host, false);
}
int khan_featurize_grad_ordered_f32(const float* xs, const float* ys, const float* zs, const int32_t* as,
                                    const int32_t* mos, const int32_t* macs, int32_t n_mols,
                                    const int32_t* sis, const float* gh, const float* gc, const float* gn,
                                    const float* go, float* gx, float* gy, float* gz,
                                    const int32_t* acs_host, const int32_t* order, const int32_t* size_classes_host,
        khan_stream_t stream)
{
    return featurize_grad_impl<float>(xs, ys, zs, as, mos, macs, n_mols, sis, gh, gc, gn, go, gx, gy, gz,
                                      acs_host, stream, order, size_classes_host, false);
}
int khan_featurize_grad_ordered_f64(const double* xs, const double* ys, const double* zs, const int32_t* as,
                                    const int32_t* mos, const int32_t* macs, int32_t n_mols,
                                    const int32_t* sis, const double* gh, const double* gc, const double* gn,
                                    const double* go, double* gx, double* gy, double* gz,
                                    const int32_t* acs_host, const int32_t* order, const int32_t* size_classes_host,
        khan_stream_t stream)
{
    return featurize_grad_impl<double>(xs, ys, zs, as, mos, macs, n_mols, sis, gh, gc, gn, go, gx, gy, gz,
                                       acs_host, stream, order, size_classes_host, false);
}
int khan_featurize_grad_inverse_ordered_f32(const float* xs, const float* ys, const float* zs, const int32_t* as,
                                            const int32_t* mos, const int32_t* macs, int32_t n_mols,
                                            const int32_t* sis, const float* x_grads, const float* y_grads,
                                            const float* z_grads, float* h, float* c, float* n, float* o,
                                            const int32_t* acs_host, const int32_t* order, const int32_t* size_classes_host,
        khan_stream_t stream)
{
    return featurize_grad_inverse_impl<float>(xs, ys, zs, as, mos, macs, n_mols, sis, x_grads, y_grads, z_grads,
                                              h, c, n, o, acs_host, stream, order, size_classes_host, false);
}
int khan_featurize_grad_inverse_ordered_f64(const double* xs, const double* ys, const double* zs, const int32_t* as,
                                            const int32_t* mos, const int32_t* macs, int32_t n_mols,
                                            const int32_t* sis, const double* x_grads, const double* y_grads,
                                            const double* z_grads, double* h, double* c, double* n, double* o,
                                            const int32_t* acs_host, const int32_t* order, const int32_t* size_classes_host,
        khan_stream_t stream)
{
    return featurize_grad_inverse_impl<double>(xs, ys, zs, as, mos, macs, n_mols, sis, x_grads, y_grads, z_grads,
                                               h, c, n, o, acs_host, stream, order, size_classes_host, false);
}

}  // extern "C"
