// C ABI of the gfx950 quaternion Conv2D / Dense engine: descriptor checks, tile planning, filter
// packing and kernel dispatch.  See include/phx_qconv.h for the contract.
#include "../../include/phx_qconv.h"

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstdint>
#include <cstring>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "phx_launch.h"
#include "phx_kernels_pw16.h"

// Scratch memory of phx_qconv2d_fwd_noalloc: a device-resident array of the code object (every GPU the library
// runs on holds its own copy until the process ends).  In host code this name is only a handle for
// hipGetSymbolAddress; the device address it stands for is looked up once per device (device_state) and that
// pointer, never the name, is what kernels and copies receive.
static __device__ __align__(256) unsigned char scratch[PHX_NOALLOC_SCRATCH_BYTES];

namespace phx {

// Developer overrides of the planner (kernel tuning experiments and the tests that pin a kernel variant), read
// from the environment once; phx_tuning_reload() reads them again and forgets the cached plans.
struct Tuning {
    int tile_wco = 0, tile_ntw = 0;   // PHX_TUNE_TILE="wco,ntw"
    bool flat = false, noflat = false, nopw = false, pw8 = false, zi8 = false, wg8 = false, nos2d = false, noearly = false, norealx = false, nosub = false, oldplan = false;
    bool nopwx = false;               // PHX_TUNE_NOPWX: pointwise fp16 problems stay on the staged-window kernels
    bool nohalf = false;              // PHX_TUNE_NOHALF: the pointwise streaming kernel never cuts items in two
    bool nopwr = false;               // PHX_TUNE_NOPWR: pointwise fp16 problems with small filters stay on the streaming kernel
    bool pwrall = false;              // PHX_TUNE_PWRALL: ... and every problem that kernel can run goes to it (not only those of at most 32 output channels)
    bool nowincl = false;             // PHX_TUNE_NOWINCL: channels-last windowed problems go through the transposes
    bool nogroupbatch = false;        // PHX_TUNE_NOGROUPBATCH: a grouped convolution runs group after group
    double wg_kpw = 0.01;             // PHX_TUNE_WGKPW: how much the fp32 filter-gradient planner favours larger pixel tiles on small images (see plan_wgrad_f32)
    int thin_max32 = 64;              // PHX_TUNE_THIN_MAX32: the same bound for passes in fp32 arithmetic (x4 for the filter gradient); PHX_TUNE_THIN_MAX=0 zeroes it too
    int thin_max = 4;                 // PHX_TUNE_THIN_MAX: most input x output channels per group that run on the vector-ALU kernels for thin groups (0 = never)
    int dilphase_min = 160;           // PHX_TUNE_DILPHASE_MIN: forward / input-gradient passes whose dilated window has more positions than this run by dilation phases
    int wgphase = -1;                 // PHX_TUNE_WGPHASE: 1 = every strided filter gradient with several taps runs by tap classes, 0 = none (unset: wgrad_by_classes)
    bool nobands = false;             // PHX_TUNE_NOBANDS: large filter windows are not cut into tap bands
    bool nopatch = false;             // PHX_TUNE_NOPATCH: convolutions whose stride equals their filter extent stay on the windowed kernels
    bool patchall = false;            // PHX_TUNE_PATCHALL: every pass of every such convolution runs on patches (not only where that was measured to gain)
    bool nodilphase = false;          // PHX_TUNE_NODILPHASE: dilated convolutions beyond the staging limit stay on the vector-ALU kernels
    int kslices = -1;                 // PHX_TUNE_KSLICES: reduction slices of a forward / input-gradient pass (0 = never, unset = by the rule of corr_slices)
    bool nodensecl = false;           // PHX_TUNE_NODENSECL: Dense never runs as a channels-last pointwise convolution
    bool nomerge = false;             // PHX_TUNE_NOMERGE: groups are never merged into block-diagonal ones
    bool direct = false;              // PHX_TUNE_DIRECT: every convolution those kernels can run goes to them (an independent path to check the matrix-core kernels against)
    bool thin_notile = false;         // PHX_TUNE_THIN_NOTILE: ... and never on the kernel that stages window tiles in LDS
    int wincl_max = 3072;             // PHX_TUNE_WINCL_MAX: largest channels x taps that runs on channels-last tensors directly
    bool nosmalldense = false;        // PHX_TUNE_NOSMALLDENSE: small Dense problems stay on the matrix-core kernels
    int vec = 0;                      // PHX_TUNE_VEC (0 = unset)
    int wgs = 0;                      // PHX_TUNE_WGS (0 = unset)
    int wg_mt = 0, wg_nt = 0;         // PHX_TUNE_WG="mt,nt"
    int wg_tpw = 0;                   // PHX_TUNE_WGTPW: taps per workgroup of the fp16 filter gradient (1 = no shared gradient tile)
    int phase = -1;                   // PHX_TUNE_PHASE (-1 = unset)
    int verbose = 0;                  // UPSTRIDE_VERBOSE (src/backend/backend.cc:45-48)
    void read() {
        *this = Tuning();
        if (const char* t = std::getenv("PHX_TUNE_TILE")) sscanf(t, "%d,%d", &tile_wco, &tile_ntw);
        flat = getenv("PHX_TUNE_FLAT") != nullptr;
        noflat = getenv("PHX_TUNE_NOFLAT") != nullptr;
        nopw = getenv("PHX_TUNE_NOPW") != nullptr;
        pw8 = getenv("PHX_TUNE_PW8") != nullptr;
        zi8 = getenv("PHX_TUNE_ZI8") != nullptr;
        wg8 = getenv("PHX_TUNE_WG8") != nullptr;
        nos2d = getenv("PHX_TUNE_NOS2D") != nullptr;
        noearly = getenv("PHX_TUNE_NOEARLY") != nullptr;
        norealx = getenv("PHX_TUNE_NOREALX") != nullptr;
        nosub = getenv("PHX_TUNE_NOSUB") != nullptr;
        oldplan = getenv("PHX_TUNE_OLDPLAN") != nullptr;
        nopwx = getenv("PHX_TUNE_NOPWX") != nullptr;
        nohalf = getenv("PHX_TUNE_NOHALF") != nullptr;
        nopwr = getenv("PHX_TUNE_NOPWR") != nullptr;
        pwrall = getenv("PHX_TUNE_PWRALL") != nullptr;
        nowincl = getenv("PHX_TUNE_NOWINCL") != nullptr;
        nogroupbatch = getenv("PHX_TUNE_NOGROUPBATCH") != nullptr;
        if (const char* e = getenv("PHX_TUNE_WINCL_MAX")) wincl_max = atoi(e);
        if (const char* e = getenv("PHX_TUNE_THIN_MAX")) { thin_max = atoi(e); if (thin_max == 0) thin_max32 = 0; }
        if (const char* e = getenv("PHX_TUNE_THIN_MAX32")) thin_max32 = atoi(e);
        if (const char* e = getenv("PHX_TUNE_WGKPW")) wg_kpw = atof(e);
        thin_notile = getenv("PHX_TUNE_THIN_NOTILE") != nullptr;
        direct = getenv("PHX_TUNE_DIRECT") != nullptr;
        nomerge = getenv("PHX_TUNE_NOMERGE") != nullptr;
        nodensecl = getenv("PHX_TUNE_NODENSECL") != nullptr;
        if (const char* e = getenv("PHX_TUNE_KSLICES")) kslices = atoi(e);
        nodilphase = getenv("PHX_TUNE_NODILPHASE") != nullptr;
        nopatch = getenv("PHX_TUNE_NOPATCH") != nullptr;
        nobands = getenv("PHX_TUNE_NOBANDS") != nullptr;
        patchall = getenv("PHX_TUNE_PATCHALL") != nullptr;
        if (const char* e = getenv("PHX_TUNE_WGPHASE")) wgphase = atoi(e) != 0;
        if (const char* e = getenv("PHX_TUNE_DILPHASE_MIN")) dilphase_min = atoi(e);
        nosmalldense = getenv("PHX_TUNE_NOSMALLDENSE") != nullptr;
        if (const char* e = getenv("PHX_TUNE_VEC")) vec = atoi(e);
        if (const char* e = getenv("PHX_TUNE_WGS")) wgs = atoi(e);
        if (const char* e = getenv("PHX_TUNE_WG")) sscanf(e, "%d,%d", &wg_mt, &wg_nt);
        if (const char* e = getenv("PHX_TUNE_WGTPW")) wg_tpw = atoi(e);
        if (const char* e = getenv("PHX_TUNE_PHASE")) phase = atoi(e) != 0;
        if (const char* e = getenv("UPSTRIDE_VERBOSE")) verbose = (int)strtol(e, nullptr, 10);
    }
};
static Tuning g_tune;
static std::once_flag g_tune_once;
static const Tuning& tune() {
    std::call_once(g_tune_once, [] { g_tune.read(); });
    return g_tune;
}
bool tuning_noearly() { return tune().noearly; }
bool tuning_thin_notile() { return tune().thin_notile; }

// Plans are pure functions of the problem and the tuning overrides; they are computed once per distinct
// problem (the reference keeps its configured operations per descriptor, src/backend/op_collections.hpp:121-144)
// and kept in bounded memos: when a miss finds more than PLAN_MEMO_LIMIT entries, all but the PLAN_MEMO_KEEP most
// recently used ones are dropped (the reference's KEEP_TOP_100 policy, src/backend/op_collections.cc:21-59).
// (fixed-size keys: a lookup that hits allocates nothing)
struct PlanKey {
    int v[24];
    bool operator==(const PlanKey& o) const { return std::memcmp(v, o.v, sizeof(v)) == 0; }
};
struct PlanKeyHash {
    size_t operator()(const PlanKey& k) const {
        size_t h = 1469598103934665603ull;
        for (int x : k.v) h = (h ^ (unsigned)x) * 1099511628211ull;
        return h;
    }
};
static std::mutex g_plan_mutex;
static unsigned g_plan_generation = 0;  // bumped (under g_plan_mutex) when the tuning overrides are read again
constexpr size_t PLAN_MEMO_LIMIT = 200, PLAN_MEMO_KEEP = 100;
static std::atomic<long> g_plan_evictions{0};
static long g_plan_memo_sizes[2] = {0, 0};  // entries of the forward / input-gradient and of the filter-gradient memo

// One memo; every method is called with g_plan_mutex held.
template <typename V>
class PlanMemo {
    struct Slot { V value; unsigned long used; };
    std::unordered_map<PlanKey, Slot, PlanKeyHash> map_;
    unsigned long clock_ = 0;
    unsigned generation_ = 0;

    void collect() {
        if (map_.size() <= PLAN_MEMO_LIMIT) return;
        std::vector<unsigned long> stamps;
        stamps.reserve(map_.size());
        for (const auto& kv : map_) stamps.push_back(kv.second.used);
        std::nth_element(stamps.begin(), stamps.end() - PLAN_MEMO_KEEP, stamps.end());
        const unsigned long oldest_kept = *(stamps.end() - PLAN_MEMO_KEEP);
        for (auto it = map_.begin(); it != map_.end();) {
            if (it->second.used < oldest_kept) { it = map_.erase(it); ++g_plan_evictions; }
            else ++it;
        }
    }

public:
    // The entry of `key`, made by `make()` on a miss.
    template <typename Make>
    const V& get(const PlanKey& key, Make make) {
        if (generation_ != g_plan_generation) { map_.clear(); generation_ = g_plan_generation; }
        auto it = map_.find(key);
        if (it == map_.end()) {
            collect();
            it = map_.emplace(key, Slot{make(), 0}).first;
        }
        it->second.used = ++clock_;
        return it->second.value;
    }
    size_t size() const { return map_.size(); }
};
// Kernels that need more dynamic LDS than the default 64 KiB (see phx_launch.h)
static std::vector<const void*>& big_lds_kernels() {
    static std::vector<const void*> v;
    return v;
}
bool register_big_lds_kernel(const void* fn) {
    big_lds_kernels().push_back(fn);
    return true;
}

// Per-device set-up, done once per device by phx_init() or by the first compute call made with that device
// current: the dynamic-LDS opt-in of every kernel variant that needs it (never done inside a launch, which may
// sit in a stream capture) and the device address of the built-in scratch array.
struct DeviceState {
    std::atomic<int> ready{0};  // 0 = not set up, 1 = ready, -1 = set-up failed
    int cu_count = 256;         // compute units (persistent kernels size their grids by it)
    void* scratch_ptr = nullptr;
};
constexpr int MAX_DEVICES = 64;
static DeviceState g_devices[MAX_DEVICES];
static std::mutex g_device_mutex;

// packed filters, partial sums and rearranged tensors are read and written as 16-byte vectors
static bool misaligned_workspace(const void* ws) { return (reinterpret_cast<uintptr_t>(ws) & 15) != 0; }

static int device_state(DeviceState** out) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) { (void)hipGetLastError(); return PHX_ERR_RUNTIME; }
    DeviceState& d = g_devices[dev];
    if (d.ready.load(std::memory_order_acquire) != 1) {
        std::lock_guard<std::mutex> lock(g_device_mutex);
        if (d.ready.load(std::memory_order_relaxed) != 1) {
            // A kernel whose opt-in fails (a device with less LDS) is the only one affected: its launch reports the
            // error, every other path runs.  Nothing is latched on failure: the next call tries again.
            bool all = true;
            for (const void* fn : big_lds_kernels())
                if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess) {
                    (void)hipGetLastError();
                    all = false;
                }
            int cus = 0;
            if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cus > 0) d.cu_count = cus;
            else (void)hipGetLastError();
            // (the built-in scratch array serves phx_qconv2d_fwd_noalloc alone, which reports a missing address itself)
            void* ptr = nullptr;
            if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess) { (void)hipGetLastError(); ptr = nullptr; }
            d.scratch_ptr = ptr;
            if (all && ptr) d.ready.store(1, std::memory_order_release);
        }
    }
    if (out) *out = &d;
    return PHX_OK;
}

static thread_local const char* g_last_kernel = "";
static thread_local char g_name_buf[160];
static thread_local const char* g_name_prefix = "";  // "s2d_" while a rewritten problem runs
static thread_local bool g_window_cl = false;        // run_corr reads and writes channels-last tensors (see nhwc_window_native)
// All groups of a grouped convolution in one launch per kernel (see group_batchable): the number of groups and the
// bytes from one group's slice of the caller's tensors to the next group's.  The runners below give every kernel a
// grid row per group and these steps (their own packed images and partial sums lie group after group in the workspace).
struct GroupBatch {
    int n = 1;
    size_t x = 0, y = 0, w = 0, b = 0;
};
static thread_local GroupBatch g_batch;
// (kernel labels of launches that run every group carry the number of groups)
static thread_local int g_name_suffix_merged = 0;  // m while groups merged m at a time run (see merged_groups)
static void label_groups(int groups) {
    size_t len = strlen(g_name_buf);
    if (groups > 1 && len < sizeof(g_name_buf)) snprintf(g_name_buf + len, sizeof(g_name_buf) - len, "_groups%d", groups);
    len = strlen(g_name_buf);
    if (g_name_suffix_merged && len < sizeof(g_name_buf))
        snprintf(g_name_buf + len, sizeof(g_name_buf) - len, "_merged%d", g_name_suffix_merged);
}
static const void* at_bytes(const void* ptr, size_t off) { return ptr ? static_cast<const char*>(ptr) + off : nullptr; }
static void* at_bytes(void* ptr, size_t off) { return ptr ? static_cast<char*>(ptr) + off : nullptr; }

// Filters packed ahead of the passes that use them (phx_qconv2d_pack_filters and the *_prepacked entry points).
// The forward and input-gradient code paths run as always, and this thread's session tells the places that pack
// what to do instead: SIZE adds up the bytes the packed images take, RECORD notes every packing call as a job of one
// combined launch (and launches nothing else), USE skips the packing and reads the images where RECORD put them.
// The same descriptor walks the same path in all three, so the images are found by their running offset.
struct PackSession {
    enum Mode { OFF, SIZE, RECORD, USE };
    Mode mode = OFF;
    char* base = nullptr;
    size_t capacity = 0, offset = 0;
    hipStream_t st = nullptr;
    PackJobs jobs{};
    bool dry() const { return mode == SIZE || mode == RECORD; }
};
static thread_local PackSession g_pack;

struct PackSessionScope {  // a session lasts for one entry-point call
    PackSessionScope(PackSession::Mode m, void* base, size_t capacity, hipStream_t st) {
        g_pack.mode = m; g_pack.base = static_cast<char*>(base); g_pack.capacity = capacity; g_pack.offset = 0; g_pack.st = st;
    }
    ~PackSessionScope() { g_pack.mode = PackSession::OFF; g_pack.base = nullptr; g_pack.capacity = g_pack.offset = 0; }
};

// An input-gradient call that adds a tensor to its result (phx_qconv2d_bwd_data_add): the kernel that writes the
// caller's dx adds it in its epilogue if it can and says so here; otherwise a separate pass adds it afterwards.
struct Addend {
    const void* ptr = nullptr;
    const void* dx = nullptr;  // the tensor the addend belongs to: only the kernel that writes THAT may take it
    bool fused = false;
};
static thread_local Addend g_addend;

static int flush_pack_jobs() {
    const int rc = launch_pack_jobs(g_pack.jobs, g_pack.st);
    g_pack.jobs.n = 0;
    return rc == 0 ? PHX_OK : PHX_ERR_NOT_SUPPORTED;
}

// Where a run's packed filters live and who packs them.  dst: the image's address (the workspace outside a
// session); pack_now: the caller launches its packing kernel as usual; compute: the caller goes on to its kernels.
struct PackSlot {
    void* dst;
    bool pack_now, compute;
    int rc;
};
static PackSlot pack_slot(void* ws, size_t ws_bytes, size_t image_bytes) {
    PackSession& s = g_pack;
    if (s.mode == PackSession::OFF) {
        if (ws_bytes < image_bytes || !ws) return {nullptr, false, false, PHX_ERR_WORKSPACE};
        return {ws, true, true, PHX_OK};
    }
    const size_t off = s.offset;
    s.offset += (image_bytes + 255) / 256 * 256;
    if (s.mode == PackSession::SIZE) return {nullptr, false, false, PHX_OK};
    if (s.offset > s.capacity || !s.base) return {nullptr, false, false, PHX_ERR_WORKSPACE};
    return {s.base + off, false, s.mode == PackSession::USE, PHX_OK};
}

// RECORD: one more job for the combined launch (a full list is launched and started anew)
static int record_pack_job(PackJob j, long items) {
    PackSession& s = g_pack;
    if (s.mode != PackSession::RECORD) return PHX_OK;
    if (s.jobs.n == PACK_JOBS_MAX)
        if (const int rc = flush_pack_jobs()) return rc;
    j.block0 = s.jobs.n ? s.jobs.job[s.jobs.n - 1].block0 + s.jobs.job[s.jobs.n - 1].nblocks : 0;
    j.nblocks = (int)std::max<long>(1, std::min<long>((items + WG_THREADS - 1) / WG_THREADS, 1024));
    s.jobs.job[s.jobs.n++] = j;
    return PHX_OK;
}

// optional event pairs around the dominant kernel of each call (see phx_profile_enable)
struct ProfileState {
    std::vector<hipEvent_t> ev;  // 2 per slot
    int used = 0;
    bool on = false;
};
static ProfileState g_prof;  // process-wide: frameworks run backward passes on their own threads
static std::mutex g_prof_mutex;

struct KernelTimer {
    hipStream_t st;
    int slot;
    explicit KernelTimer(hipStream_t s) : st(s), slot(-1) {
        if (!g_prof.on) return;
        // no event records into a stream capture: a captured graph would replay them against events of this run
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(st, &cs) != hipSuccess) { (void)hipGetLastError(); return; }
        if (cs != hipStreamCaptureStatusNone) return;
        std::lock_guard<std::mutex> lock(g_prof_mutex);
        if (2 * (g_prof.used + 1) <= (int)g_prof.ev.size()) {
            slot = g_prof.used++;
            (void)hipEventRecord(g_prof.ev[2 * slot], st);
        }
    }
    ~KernelTimer() {
        if (slot >= 0) (void)hipEventRecord(g_prof.ev[2 * slot + 1], st);
    }
};

#define PHX_HIP(call)                                              \
    do {                                                           \
        hipError_t e_ = (call);                                    \
        if (e_ != hipSuccess) { (void)hipGetLastError(); return PHX_ERR_RUNTIME; } \
    } while (0)

static inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
static inline int cdiv(int a, int b) { return (a + b - 1) / b; }

// Filter addressing: element (r, o, i, kh, kw) at r*wcs + o*so + i*si + kh*skh + kw*skw
struct FilterStrides {
    long wcs, so, si, skh, skw;
};

// One quaternion correlation problem in the engine's internal terms
struct Problem {
    int dtype, mode, policy;
    int n, ci, co, h, w, kh, kw, sh, sw, dh, dw, pt, pl, pb, pr, ho, wo;
    FilterStrides fs;
    bool has_bias;
    bool real_input;  // x (and dx) are real-valued [n, ci, h, w]: imaginary components are zero and not stored
    // Grouped convolution: ci / co above are one group's channels, the tensors hold ci_mem / co_mem channels per
    // image and `groups` such slices side by side (ci_mem == ci, co_mem == co without groups)
    int groups, ci_mem, co_mem;
    bool nhwc;  // the caller's activation tensors are channels-last: [rows, h, w, channels]
    bool banded = false;  // a band of a larger filter's taps (see tap_bands): pads may be negative, and no rewrite applies
};

static int out_size(int in, int k, int d, int s, int before, int after) {
    const int eff = (k - 1) * d + 1;
    return (in + before + after - eff + s) / s;
}

static int problem_from_conv(const phx_qconv_desc* d, Problem& p) {
    if (!d) return PHX_ERR_INVALID_ARGUMENT;
    if (d->dtype != PHX_F32 && d->dtype != PHX_F16) return PHX_ERR_INVALID_ARGUMENT;
    if (d->product_mode != PHX_PRODUCT_16 && d->product_mode != PHX_PRODUCT_8) return PHX_ERR_INVALID_ARGUMENT;
    if (d->fp16_policy < PHX_FP16_FULL32 || d->fp16_policy > PHX_FP16_FULL16) return PHX_ERR_INVALID_ARGUMENT;
    if (d->filter_layout != PHX_OIHW && d->filter_layout != PHX_OHWI && d->filter_layout != PHX_HWIO)
        return PHX_ERR_INVALID_ARGUMENT;
    if (d->n < 0 || d->ci <= 0 || d->co <= 0 || d->h < 0 || d->w < 0 || d->kh <= 0 || d->kw <= 0)
        return PHX_ERR_INVALID_ARGUMENT;
    if (d->stride_h <= 0 || d->stride_w <= 0 || d->dilation_h <= 0 || d->dilation_w <= 0)
        return PHX_ERR_INVALID_ARGUMENT;
    if (d->pad_top < 0 || d->pad_left < 0 || d->pad_bottom < 0 || d->pad_right < 0) return PHX_ERR_INVALID_ARGUMENT;
    if (d->real_input != 0 && d->real_input != 1) return PHX_ERR_INVALID_ARGUMENT;
    // "Bias addition is not supported for type0 inputs" (src/conv2d.hpp:125-127)
    if (d->real_input && d->has_bias) return PHX_ERR_INVALID_ARGUMENT;
    if (d->data_format != PHX_NCHW && d->data_format != PHX_NHWC) return PHX_ERR_INVALID_ARGUMENT;
    if (d->algebra < PHX_QUATERNION || d->algebra > PHX_GA_300) return PHX_ERR_INVALID_ARGUMENT;
    const int groups = d->groups > 1 ? d->groups : 1;
    if (d->ci % groups || d->co % groups) return PHX_ERR_INVALID_ARGUMENT;
    p.dtype = d->dtype;
    p.mode = d->product_mode;
    p.policy = d->fp16_policy;
    p.groups = groups; p.ci_mem = d->ci; p.co_mem = d->co;
    p.n = d->n; p.ci = d->ci / groups; p.co = d->co / groups; p.h = d->h; p.w = d->w; p.kh = d->kh; p.kw = d->kw;
    p.sh = d->stride_h; p.sw = d->stride_w; p.dh = d->dilation_h; p.dw = d->dilation_w;
    p.pt = d->pad_top; p.pl = d->pad_left; p.pb = d->pad_bottom; p.pr = d->pad_right;
    p.ho = out_size(p.h, p.kh, p.dh, p.sh, p.pt, p.pb);
    p.wo = out_size(p.w, p.kw, p.dw, p.sw, p.pl, p.pr);
    if ((p.h > 0 && p.ho <= 0) || (p.w > 0 && p.wo <= 0)) return PHX_ERR_INVALID_ARGUMENT;
    const long taps = (long)p.kh * p.kw;
    p.fs.wcs = (long)p.co_mem * p.ci * taps;  // filter [4][co_mem][ci per group][kh][kw]
    if (d->filter_layout == PHX_OIHW) {
        p.fs.so = p.ci * taps; p.fs.si = taps; p.fs.skh = p.kw; p.fs.skw = 1;
    } else if (d->filter_layout == PHX_OHWI) {
        p.fs.so = taps * p.ci; p.fs.si = 1; p.fs.skh = (long)p.kw * p.ci; p.fs.skw = p.ci;
    } else {  // HWIO: [kh][kw][ci per group][co_mem]
        p.fs.so = 1; p.fs.si = p.co_mem; p.fs.skw = (long)p.ci * p.co_mem; p.fs.skh = (long)p.kw * p.ci * p.co_mem;
    }
    p.has_bias = d->has_bias != 0;
    p.real_input = d->real_input != 0;
    p.nhwc = d->data_format == PHX_NHWC;
    return PHX_OK;
}

static int problem_from_dense(const phx_qdense_desc* d, Problem& p) {
    if (!d) return PHX_ERR_INVALID_ARGUMENT;
    if (d->dtype != PHX_F32 && d->dtype != PHX_F16) return PHX_ERR_INVALID_ARGUMENT;
    if (d->product_mode != PHX_PRODUCT_16 && d->product_mode != PHX_PRODUCT_8) return PHX_ERR_INVALID_ARGUMENT;
    if (d->fp16_policy < PHX_FP16_FULL32 || d->fp16_policy > PHX_FP16_FULL16) return PHX_ERR_INVALID_ARGUMENT;
    if (d->n < 0 || d->ni <= 0 || d->no <= 0) return PHX_ERR_INVALID_ARGUMENT;
    if (d->filter_layout != PHX_IO && d->filter_layout != PHX_OI) return PHX_ERR_INVALID_ARGUMENT;
    if (d->algebra != PHX_QUATERNION) return PHX_ERR_INVALID_ARGUMENT;
    p.dtype = d->dtype; p.mode = d->product_mode; p.policy = d->fp16_policy;
    p.n = d->n; p.ci = d->ni; p.co = d->no; p.h = p.w = 1; p.kh = p.kw = 1;
    p.sh = p.sw = p.dh = p.dw = 1; p.pt = p.pl = p.pb = p.pr = 0; p.ho = p.wo = 1;
    // layout IO: w[r][i][o]; OI: w[r][o][i]
    p.fs.wcs = (long)p.ci * p.co; p.fs.skh = 0; p.fs.skw = 0;
    if (d->filter_layout == PHX_IO) { p.fs.so = 1; p.fs.si = p.co; }
    else { p.fs.so = p.ci; p.fs.si = 1; }
    p.has_bias = d->has_bias != 0;
    p.real_input = false;
    p.groups = 1; p.ci_mem = p.ci; p.co_mem = p.co;
    p.nhwc = false;
    return PHX_OK;
}

// UPSTRIDE_VERBOSE > 0 (src/backend/backend.cc:45-62, the reference's UPSTRIDE_SAYS): one line per kernel
// dispatch naming the product mode asked for, the fp16 policy and the kernel variant chosen
static void say(const Problem& p, const char* pass) {
    if (tune().verbose <= 0) return;
    static const char* const policies[] = {"fp32", "backward32", "full16"};
    fprintf(stderr, "[upstride] quaternion %s: product mode %d, fp16 policy %s, kernel %s\n", pass, p.mode,
            p.dtype == PHX_F16 ? policies[p.policy] : "n/a (fp32 tensors)", g_last_kernel);
}

static bool is_empty(const Problem& p) { return p.n == 0 || p.h == 0 || p.w == 0; }
// the problem works on a slice of its tensors' channels (one of several groups, or what is left of them): the paths
// that rearrange whole tensors do not apply
static bool channel_slices(const Problem& p) { return p.groups > 1 || p.ci_mem != p.ci || p.co_mem != p.co; }

static bool is_pointwise_unit(const Problem& p) {
    return p.kh == 1 && p.kw == 1 && p.sh == 1 && p.sw == 1 && !p.pt && !p.pl && !p.pb && !p.pr;
}

// A pointwise, unit-stride, unpadded convolution sees each image plane as one long row
static Problem flatten_pointwise(const Problem& p) {
    Problem f = p;
    if (is_pointwise_unit(p)) {
        f.w = p.h * p.w; f.h = 1;
        f.wo = p.ho * p.wo; f.ho = 1;
    }
    return f;
}

// -------------------------------------------------------------------------------------------
// Correlation view shared by forward and input-gradient: out[N][Cout][Hout][Wout] from
// in[N][Cin][Hin][Win] (seen through zero insertion uh, uw), unit stride unless forward.
// -------------------------------------------------------------------------------------------
struct Corr {
    int N, Cin, Hin, Win, Cout, Hout, Wout;
    int Kh, Kw, sh, sw, dh, dw, pt, pl, uh, uw;
    // input gradient: tap (u, v) of the correlation is filter tap (khm - u*khs, kwm - v*kws); the plain mirrored
    // filter has khm = Kh-1, khs = 1
    int khm, khs, kwm, kws;
    int ncomp;  // components of the input present in memory: 4, or 1 for the forward pass on a real-valued input
};

static Corr corr_forward(const Problem& p) {
    Corr c{p.n, p.ci, p.h, p.w, p.co, p.ho, p.wo, p.kh, p.kw, p.sh, p.sw, p.dh, p.dw, p.pt, p.pl, 1, 1, p.kh - 1, 1, p.kw - 1, 1};
    if (p.kh == 1 && p.kw == 1 && p.sh == 1 && p.sw == 1 && !p.pt && !p.pl && !p.pb && !p.pr) {
        c.Win = p.h * p.w; c.Hin = 1; c.Wout = p.ho * p.wo; c.Hout = 1;  // pointwise: one long row per image
    }
    c.ncomp = p.real_input ? 1 : 4;
    return c;
}

static Corr corr_dgrad(const Problem& p) {
    Corr c{p.n, p.co, p.ho, p.wo, p.ci, p.h, p.w, p.kh, p.kw, 1, 1, p.dh, p.dw,
           (p.kh - 1) * p.dh - p.pt, (p.kw - 1) * p.dw - p.pl, p.sh, p.sw, p.kh - 1, 1, p.kw - 1, 1};
    if (p.kh == 1 && p.kw == 1 && p.sh == 1 && p.sw == 1 && !p.pt && !p.pl && !p.pb && !p.pr) {
        c.Win = p.ho * p.wo; c.Hin = 1; c.Wout = p.h * p.w; c.Hout = 1;
    }
    c.ncomp = 4;
    return c;
}

struct FwdPlan {
    int WCO, NTW, BN;
    int kmode;               // product formulation the kernel runs in (see plan_corr)
    int CK, P2LOG;           // channels per chunk and log2 staging positions of the kernel variant
    bool lds_filters;        // fp16 MFMA, 16-product, more than one tap: filters go through LDS
    int ngroups;             // tap groups per chunk in that case
    bool vstage;             // fp32 MFMA: window rows widened to a multiple of 4, staged as 4-position vectors
    bool pairs;              // fp16 MFMA: window rows widened to even columns, staged as position pairs
    bool chunks;             // fp16 MFMA, filters in LDS: window rows widened to a multiple of 8, staged as chunks
    int NB, TH, TW, HTH, HTW, HP, HPp;
    int tiles_n, tiles_h, tiles_w, co_tiles, nchunks;
    size_t lds_bytes, wpk_bytes;
    int wgs;
    int tall;                // flat tiling (row distance of the images in the tall image), 0 = rectangular tiles
    int pwx;                 // pointwise kernel with raw operand copies (phx_kernels_pw16.h): its WCO, 0 = not that kernel
    int pwx_steps;           // ... its K steps of 16 channels
};


constexpr int LDS_FLOATS_MAX = 16384;  // 64 KiB: two workgroups per CU

static bool plan_forward(const Corr& c, int mode, bool f16mfma, FwdPlan& best, bool pointwise = false) {
    double best_score = -1.0;
    // fp16 MFMA with filters in LDS: stage activations as aligned pairs when rows are even
    // filters through LDS: 16-product always, 8-product where the chunk staging applies
    // the vector staging forms copy runs of stored positions: no zero insertion along either axis
    const bool dense_window = c.uh == 1 && c.uw == 1;
    const bool ldsk = f16mfma && c.Kh * c.Kw > 1 && (mode == 16 || dense_window);
    const bool chunks = ldsk && dense_window;
    const bool pairs = f16mfma && !chunks && (c.Win % 2 == 0) && dense_window;
    const bool vstage = !f16mfma && dense_window;
    best.pairs = pairs; best.chunks = chunks; best.vstage = vstage;
    const int wcos[3] = {1, 2, 4};
    // PHX_TUNE_TILE="wco,ntw" pins the workgroup shape (kernel tuning experiments)
    const int force_wco = tune().tile_wco, force_ntw = tune().tile_ntw;
    const bool force_flat = tune().flat;
    for (int wi = 0; wi < 3; ++wi) {
        const int WCO = wcos[wi];
        if (force_wco && WCO != force_wco) continue;
        if (WCO > 1 && 32 * WCO > ((c.Cout + 31) / 32) * 32) continue;
        if (ldsk && mode == 8 && WCO > 2) continue;  // eight filter lanes: the LDS images of 4 sub-tiles do not fit
        // 8 lanes x 2 column tiles fill the whole AGPR file: only the LDS kernel is built that way
        for (int NTW = 1; NTW <= ((mode == 16 || ldsk) ? 2 : 1); ++NTW) {
            if (force_ntw && NTW != force_ntw) continue;
            const int BN = (4 / WCO) * NTW * 32;
            const int cot = cdiv(c.Cout, 32 * WCO);
            auto consider = [&](int NB, int TH, int TW, int HTH, int HTW, int tn, int th, int tw, int tall) {
                const int HP = NB * HTH * HTW;
                if (HP > 256) return;  // one staging position per thread
                const long wgs = (long)tn * th * tw * cot;
                const double eff = ((double)c.N * c.Hout * c.Wout * c.Cout) / ((double)wgs * BN * 32 * WCO);
                const double fill = (double)wgs / ((double)cdiv((int)std::min<long>(wgs, 1 << 30), 512) * 512);
                const double halo = (double)std::min(NB * TH * TW, BN) / HP;  // staged data actually used
                // (fp32 matrix cores, 16-product: two column tiles per wave measured slower than any one-tile shape --
                // 3x3, 256 channels at 14x14: 5.1 against 4.1-4.6 ms -- where only the count of workgroups favoured them)
                double score = eff * (0.25 + 0.75 * fill) * (0.9 + 0.1 * halo) *
                               (NTW == 2 ? ((!f16mfma && !tune().oldplan) ? 0.9 : 1.02) : 1.0);
                // fp16 MFMA is operand-bandwidth hungry: two column tiles per wave and two filter
                // sub-tiles per workgroup amortise LDS reads and activation staging (measured)
                // (pointwise problems, 16-product: workgroups live for a few blocks only, and two of them
                // per CU -- one column tile per wave, two filter sub-tiles -- hide each other's start and end)
                if (ldsk && pointwise && mode == 16) score *= (NTW == 1 ? 1.25 : 1.0) * (WCO == 2 ? 1.2 : 1.0);
                else if (ldsk && mode == 8) {
                    // The factorized LDS kernels hold one workgroup per CU, so their time is counted out: rounds of
                    // workgroups over the CUs (half by the whole rounds the last workgroup waits for, half by the
                    // work there is -- a last round that is partly empty still frees power and memory bandwidth) times
                    // the tile's area over the shape's throughput (measured at 128 channels, 28x28, per unit of tile
                    // area: two column tiles per wave 1.0 / 1.04 with two / one filter sub-tile, one column tile
                    // 0.79 / 0.85).  A small problem then takes the small tile that fills the CUs (64 channels at
                    // 14x14, N=64: 0.041 -> 0.032 ms per pass).
                    const double rate = NTW == 2 ? (WCO == 2 ? 1.0 : 1.04) : (WCO == 2 ? 0.79 : 0.85);
                    const double cus = 256.0;
                    const double rounds = 0.5 * std::ceil(wgs / cus) + 0.5 * (wgs / cus);
                    score = 1e6 * rate / (rounds * BN * 32.0 * WCO) * (0.9 + 0.1 * halo);
                } else if (ldsk && !pointwise && !tune().oldplan) {
                    // the 16-product LDS kernels by the same count (one column tile per wave: two workgroups share a
                    // CU at about half speed each, so the rounds are still rounds over the CUs)
                    // (measured at 128 channels 28x28 and 256 channels 14x14, N=128, per unit of tile area)
                    const double rate = NTW == 2 ? (WCO == 1 ? 1.05 : 1.0) : (WCO == 1 ? 1.05 : WCO == 2 ? 1.04 : 0.87);
                    const double cus = 256.0;
                    const double rounds = 0.5 * std::ceil(wgs / cus) + 0.5 * (wgs / cus);
                    score = 1e6 * rate / (rounds * BN * 32.0 * WCO) * (0.9 + 0.1 * halo);
                } else if (ldsk) score *= (NTW == 2 ? 1.25 : 1.0) * (WCO == 2 ? 1.08 : 1.0);
                else if (f16mfma && NTW == 2) score *= 0.8;  // that kernel drops to one workgroup per CU
                if (tall && force_flat) score *= 100.0;  // (tests: flat tiling wherever it applies)
                if (score > best_score) {
                    best_score = score;
                    best.WCO = WCO; best.NTW = NTW; best.BN = BN;
                    best.NB = NB; best.TH = TH; best.TW = TW; best.HTH = HTH; best.HTW = HTW;
                    best.HP = HP; best.HPp = HP;
                    best.tiles_n = tn; best.tiles_h = th; best.tiles_w = tw; best.co_tiles = cot;
                    best.wgs = (int)wgs;
                    best.tall = tall;
                }
            };
            // Flat tiling (chunk-staging kernels, unit stride): the images are stacked into one tall image, far
            // enough apart that no window of one reaches the rows of another, and a workgroup takes BN consecutive
            // output positions of it in row-major order: every lane works whatever the image size (a 28-wide
            // image fills 112 of 128 lanes with rectangular tiles, a 14x14 one 98 or 126 of them on 14 of 18 rows).
            // Measured: it pays where the matrix pipe is the bound (two column tiles per wave, long reductions:
            // +4-7 % at 128 channels, 28x28) and costs where workgroups are short-lived and the larger window's
            // staging shows (-7 % at 32 channels), so it is offered only to the former.
            const bool flat_pays = NTW == 2 && (long)c.Cin * c.Kh * c.Kw >= 576;
            if (chunks && !pointwise && c.sh == 1 && c.sw == 1 && (flat_pays || force_flat) &&
                !tune().noflat) {
                const int reach = (c.Hout - 1) - c.pt + (c.Kh - 1) * c.dh - (c.Hin - 1);  // rows read below the image
                const int gap = std::max(0, std::max(c.pt, reach));
                const long S = (long)c.Hin + gap;                          // row distance of the images
                const long Q = ((long)(c.N - 1) * S + c.Hout) * c.Wout;    // output positions of the tall image
                const int rows = (BN + c.Wout - 2) / c.Wout + 1;           // rows BN consecutive positions can touch
                const int HTH = rows + (c.Kh - 1) * c.dh;
                const int HTW = (c.Wout + (c.Kw - 1) * c.dw + 7) & ~7;
                if (c.Hout <= S && Q < (1L << 30))
                    consider(1, rows, c.Wout, HTH, HTW, 1, (int)cdiv((int)Q, BN), 1, (int)S);
            }
            int cand[24];
            int nc = 0;
            for (int k = 1; k <= 8; ++k) cand[nc++] = cdiv(c.Wout, k);
            cand[nc++] = 8; cand[nc++] = 16; cand[nc++] = 32; cand[nc++] = BN;
            // (long rows whose window must stay within the staging limit: fractions of the workgroup's pixels)
            cand[nc++] = BN / 2; cand[nc++] = (3 * BN) / 4; cand[nc++] = 48; cand[nc++] = 80;
            cand[nc++] = 1; cand[nc++] = 2; cand[nc++] = 3;  // (windows that take most of the staging limit by themselves)
            for (int a = 0; a < nc; ++a) {
                const int TW = std::min(cand[a], std::min(c.Wout, BN));
                if (TW <= 0) continue;
                for (int TH = 1; TH <= std::min(c.Hout, BN / TW); ++TH) {
                    int NB = 1;
                    if (TH == c.Hout && TW == c.Wout) NB = std::max(1, std::min(c.N, BN / (TH * TW)));
                    const int HTH = (TH - 1) * c.sh + (c.Kh - 1) * c.dh + 1;
                    int HTW = (TW - 1) * c.sw + (c.Kw - 1) * c.dw + 1;
                    if (pairs) HTW = (HTW + 2) & ~1;  // room for the even start column, even pitch
                    if (chunks) HTW = (HTW + 7) & ~7;  // whole 8-position chunks
                    if (vstage) HTW = (HTW + 3) & ~3;  // whole 4-position groups
                    NB = std::max(1, std::min(NB, 256 / (HTH * HTW)));  // (as many whole images as the staging limit holds)
                    consider(NB, TH, TW, HTH, HTW, cdiv(c.N, NB), cdiv(c.Hout, TH), cdiv(c.Wout, TW), 0);
                }
            }
        }
    }
    if (best_score < 0) return false;
    const int WC = (mode == 16) ? 4 : 8;
    const int taps = c.Kh * c.Kw;
    if (f16mfma) {
        // fp16 MFMA: 16-channel chunks, one 16-byte LDS entry per (component, 8-channel pack, position)
        best.CK = F16_CK;
        best.P2LOG = best.HP <= 128 ? 7 : 8;
        best.nchunks = cdiv(c.Cin, best.CK);
        if (chunks) best.HPp = F16_XPITCH;  // the chunk-staging kernels address the window with a fixed unit pitch
        best.lds_bytes = (size_t)8 * best.HPp * 16;
        best.wpk_bytes = (size_t)best.co_tiles * best.WCO * best.nchunks * taps * 64 * WC * 16;
        best.lds_filters = ldsk;
        best.ngroups = cdiv(taps, F16_TG);
        if (best.lds_filters) {
            const size_t wimg = (size_t)F16_TG * best.WCO * WC * 64 * 16;  // one filter group image
            best.lds_bytes += 2 * wimg;
            best.wpk_bytes = (size_t)best.co_tiles * best.nchunks * best.ngroups * wimg;
        }
        return true;
    }
    // fp32 MFMA: pointwise problems are bandwidth/latency bound and take as many channels per
    // chunk as 32 staging registers per thread allow; everything else uses 8-channel chunks
    best.CK = F32_CK; best.P2LOG = 8; best.lds_filters = false; best.ngroups = 0;
    if (vstage) best.HPp = (best.HP + 3) & ~3;  // 16-byte aligned LDS rows
    if (taps == 1 && c.Cin >= 32 && vstage) {
        if (best.HP <= 64) { best.CK = 32; best.P2LOG = 6; }
        else if (best.HP <= 128) { best.CK = 16; best.P2LOG = 7; }
    }
    best.nchunks = cdiv(c.Cin, best.CK);
    best.lds_bytes = (size_t)4 * best.CK * best.HPp * sizeof(float);
    // packed in 8-channel groups: nchunks * CK/8 groups per filter tile
    best.wpk_bytes = (size_t)best.co_tiles * best.WCO * best.nchunks * (best.CK / F32_CK) * taps * 4 * 64 * WC *
                     sizeof(float);
    return true;
}

// fp16 tensors use fp16 matrix-core arithmetic where UPSTRIDE_CONV_FP16_POLICY allows it for the
// pass (forward: full16 or backward32; backward: full16 only), fp32 arithmetic otherwise
static bool use_f16_mfma(const Problem& p, int pass) {
    if (p.dtype != PHX_F16) return false;
    if (pass == PHX_PASS_FWD) return p.policy == PHX_FP16_FULL16 || p.policy == PHX_FP16_BACKWARD32;
    return p.policy == PHX_FP16_FULL16;
}

// A pointwise fp16 correlation on one long row per image has a single tap, which would leave the LDS
// kernels one MFMA block per barrier.  It is run instead as a column of PW_TAPS virtual taps: window
// row r of the staged tile holds the 16-channel sub-chunk r of a 48-channel chunk, and "tap" r of the
// packed filters holds the matching filter slice.  Returns the virtual correlation (pw = its tap count).
constexpr int PW_TAPS = F16_TG;
static Corr virtual_pointwise(const Corr& c, bool f16mfma, int& pw) {
    pw = 0;
    if (!f16mfma || c.Kh * c.Kw != 1 || c.uh != 1 || c.uw != 1 || c.sh != 1 || c.sw != 1 || c.Hin != 1 || c.Hout != 1 ||
        c.pt != 0 || c.pl != 0 || c.Win != c.Wout)
        return c;
    if (tune().nopw) return c;
    pw = PW_TAPS;
    Corr v = c;
    v.Kh = PW_TAPS; v.Kw = 1; v.dh = 1;
    v.Cin = 16 * cdiv(c.Cin, 16 * PW_TAPS);  // 16 virtual channels per 48-channel chunk
    return v;
}

// plans the virtual-tap form of a pointwise correlation where it applies and fits, the plain form otherwise
// pl.kmode is the product formulation the kernel runs in.  It is the mode asked for, except for pointwise
// problems on fp16 matrix cores in 8-product mode: their workgroups live for two or three tap groups, where
// the factorized kernel (one workgroup per CU, lane arithmetic in front of every block) loses to the
// 16-product kernel with two workgroups per CU (128->128@28^2: 412 against 592 TFLOP/s real-equivalent; the
// 16<->64-channel layers of a ResNet 37-75 against 64-112).  The 8-product mode means "prefer speed"
// (src/backend/backend.hpp:36-66), so those problems run on the 16-product kernel; PHX_TUNE_PW8 keeps the
// factorized one (tests exercise it).
// Pointwise correlations on fp16 matrix cores whose planes have an even number (>= 8) of pixels run on the kernel
// with raw operand copies, in 16-product form whatever the mode asks for (the 8-product mode means "prefer speed",
// src/backend/backend.hpp:36-66, and this is the fastest pointwise kernel there is); PHX_TUNE_NOPWX keeps them on
// the staged-window kernels.
static int pwx_wco(int cout);
static bool pwx_applies(const Corr& c, bool f16mfma) {
    return f16mfma && c.Kh * c.Kw == 1 && c.uh == 1 && c.uw == 1 && c.sh == 1 && c.sw == 1 && c.Hin == 1 && c.Hout == 1 &&
           c.pt == 0 && c.pl == 0 && c.Win == c.Wout && c.Win % 2 == 0 && c.Win >= 8 && c.ncomp == 4 &&
           (long)c.N * ((c.Win + 7) / 8) < (1L << 30) && !tune().nopwx && !tune().pw8;
}

static bool plan_corr_uncached(const Corr& creal, int mode, bool f16mfma, Corr& c, FwdPlan& pl, int& pw) {
    pl.pwx = 0; pl.pwx_steps = 0;
    if (pwx_applies(creal, f16mfma)) {
        pw = 0;
        c = creal;
        pl = FwdPlan{};
        pl.kmode = 16;
        pl.pwx = pwx_wco(creal.Cout);
        pl.WCO = pl.pwx; pl.NTW = 2; pl.CK = F16_CK;
        pl.co_tiles = cdiv(creal.Cout, 32 * pl.pwx);
        pl.pwx_steps = cdiv(creal.Cin, 16);
        pl.nchunks = pl.pwx_steps;
        pl.wpk_bytes = pwx_packed_bytes(pl.pwx, pl.co_tiles, pl.pwx_steps);
        return true;
    }
    c = virtual_pointwise(creal, f16mfma, pw);
    if (pw) {
        pl.kmode = (mode == 8 && !tune().pw8) ? 16 : mode;
        if (plan_forward(c, pl.kmode, f16mfma, pl, true) && pl.lds_filters && pl.chunks) return true;
    }
    pw = 0;
    c = creal;
    // zero-inserted windows (input gradient of a strided convolution with several taps) on fp16 matrix cores:
    // the factorized kernel has no LDS-filter form for them, the 16-product kernel has (3x3 stride 2 at
    // 32-128 channels: 0.15-0.18 ms against 0.08-0.11 ms), so the 8-product mode takes that one here as well
    const bool zero_inserted = c.uh > 1 || c.uw > 1;
    pl.kmode = (f16mfma && mode == 8 && zero_inserted && c.Kh * c.Kw > 1 && !tune().zi8) ? 16 : mode;
    // Real-valued input (one stored component) on fp16 matrix cores: the factorized kernel forms its lanes from one
    // real and three zero components for nothing; the 16-product kernel is the faster one (q-ResNet-50 stem, 7x7
    // stride 2 on 3 channels by space-to-depth: 0.19 against 0.30 ms).  Skipping the twelve products with the absent
    // components as well would need a kernel variant of its own: a run-time branch around them slowed every
    // 16-product convolution by 5-15 %.
    if (f16mfma && mode == 8 && c.ncomp == 1 && !tune().zi8) pl.kmode = 16;
    // One or two 16-channel chunks to reduce over: a workgroup is mostly its start and its epilogue, which the
    // 16-product kernel has less of (four accumulators to write out instead of eight lanes to merge, two workgroups
    // per CU with one column tile per wave).  3x3 on 16 channels at 56x56, N=64: 0.063 -> 0.047 ms; on 32 at 28x28:
    // 0.029 -> 0.028; from 64 channels on the factorized kernel wins (14x14: 0.032 against 0.033).
    // (with 25 taps the halved products count again: 5x5 on 24 channels 0.031 against 0.034 ms)
    if (f16mfma && mode == 8 && c.Kh * c.Kw > 1 && c.Kh * c.Kw <= 9 && c.Cin <= 32 && !tune().zi8) pl.kmode = 16;
    return plan_forward(c, pl.kmode, f16mfma, pl);
}

struct CorrPlan {
    Corr c;
    FwdPlan pl;
    int pw;
    bool ok;
};

static bool plan_corr(const Corr& creal, int mode, bool f16mfma, Corr& c, FwdPlan& pl, int& pw) {
    static PlanMemo<CorrPlan> memo;
    static_assert(sizeof(Corr) == 22 * sizeof(int), "Corr is hashed as raw ints: no padding allowed");
    PlanKey key{};
    std::memcpy(key.v, &creal, sizeof(Corr));
    key.v[22] = mode;
    key.v[23] = f16mfma;
    std::lock_guard<std::mutex> lock(g_plan_mutex);
    const CorrPlan& hit = memo.get(key, [&] {
        CorrPlan cp{};
        cp.ok = plan_corr_uncached(creal, mode, f16mfma, cp.c, cp.pl, cp.pw);
        return cp;
    });
    g_plan_memo_sizes[0] = (long)memo.size();
    c = hit.c; pl = hit.pl; pw = hit.pw;
    return hit.ok;
}

static int record_pwx_job(const PackArgs& pa, int map, int wco, int nsteps) {
    PackJob j{};
    j.a = pa; j.kind = PACK_PWX; j.mode = 16; j.map = map; j.WCO = wco; j.nsteps = nsteps;
    return record_pack_job(j, (long)pa.row_tiles * nsteps * wco * 4 * 64);
}

static int run_pwx(const Problem& p, const Corr& c, const FwdPlan& pl, int map, hipStream_t st, const void* in, const void* w,
                   const void* bias, void* out, void* ws, size_t ws_bytes) {
    const GroupBatch gb = g_batch;
    const size_t image = align_up(pl.wpk_bytes, 256);  // (group after group where one launch runs them all)
    const PackSlot slot = pack_slot(ws, ws_bytes, gb.n > 1 ? image * gb.n : pl.wpk_bytes);
    if (slot.rc != PHX_OK) return slot.rc;
    ws = slot.dst;
    PackArgs pa{};
    pa.groups = gb.n; pa.g_w = (long)gb.w; pa.g_out = (long)image;
    pa.w = w; pa.out = ws;
    pa.wcs = p.fs.wcs; pa.so = p.fs.so; pa.si = p.fs.si; pa.skh = p.fs.skh; pa.skw = p.fs.skw;
    pa.Co = p.co; pa.Ci = p.ci; pa.Kh = 1; pa.Kw = 1;
    pa.khm = c.khm; pa.khs = c.khs; pa.kwm = c.kwm; pa.kws = c.kws;
    pa.rows = c.Cout; pa.red = c.Cin; pa.row_tiles = pl.co_tiles; pa.nchunks = pl.pwx_steps;
    if (slot.pack_now && launch_pack_filters_pwx(map, pl.pwx, pl.pwx_steps, pa, st) != 0) return PHX_ERR_NOT_SUPPORTED;
    for (int g = 0; g < gb.n; ++g) {  // (the combined packing launch takes one job per image)
        PackArgs one = pa;
        one.groups = 1;
        one.w = at_bytes(pa.w, g * gb.w);
        one.out = at_bytes(pa.out, g * image);
        if (const int rrc = record_pwx_job(one, map, pl.pwx, pl.pwx_steps)) return rrc;
    }
    if (!slot.compute) return PHX_OK;
    DeviceState* dev = nullptr;
    if (const int rc = device_state(&dev)) return rc;
    const int cin_mem = (map == MAP_FWD) ? p.ci_mem : p.co_mem, cout_mem = (map == MAP_FWD) ? p.co_mem : p.ci_mem;
    PwxArgs a{};
    a.in = static_cast<const _Float16*>(in); a.in_cs = (long)c.N * cin_mem * c.Win;
    a.wpk = static_cast<const f16x8*>(ws); a.bias = static_cast<const _Float16*>(bias);
    a.out = static_cast<_Float16*>(out); a.out_cs = (long)c.N * cout_mem * c.Wout;
    a.N = c.N; a.Cin = c.Cin; a.CinS = cin_mem; a.Cout = c.Cout; a.CoutS = cout_mem; a.HW = c.Win;
    a.GI = cdiv(c.Win, 8); a.TGp = c.N * a.GI;
    a.co_tiles = pl.co_tiles; a.nsteps = pl.pwx_steps;
    a.groups = gb.n; a.g_in = (long)(map == MAP_FWD ? gb.x : gb.y); a.g_w = (long)image; a.g_bias = (long)gb.b;
    a.g_out = (long)(map == MAP_FWD ? gb.y : gb.x);
    // (a grouped convolution runs this once per group on a channel slice: only an ungrouped call covers the whole
    // addend with one launch, the groups leave it to the separate pass)
    if (map == MAP_DGRAD && g_addend.ptr && out == g_addend.dx && !g_addend.fused && p.groups == 1) {
        a.addend = static_cast<const _Float16*>(g_addend.ptr);
        g_addend.fused = true;
    }
    // Small filters (the packed image and the waves' copy rings fit 160 KiB of LDS, one output-channel tile, whole K
    // steps, at least two, plane size a multiple of 8) can run on the kernel that keeps the filter resident and never
    // synchronises its waves (phx_kernels_pwr16.h); it reads the packed image the streaming kernel reads, so
    // prepacked filters serve both.  Measured against the streaming kernel (N=64; forward, us): at most 32 output
    // channels 64->32 @56x56 42 against 56, 32->32 @56x56 24 against 36, 64->16 @56x56 29 against 37, 128->32 @28x28 19
    // against 23 -- there the streaming kernel's workgroup tile is 256 pixels wide and stores its quads directly;
    // wider outputs 64->64 @56x56 54 against 50-62, 128->64 @28x28 26 against 24, 64->128 @28x28 37 against 29,
    // 128->128 @28x28 (N=128) 78-81 against 76-79.  So it takes the problems of at most 32 output channels;
    // PHX_TUNE_PWRALL sends it everything it can run.
    if (!tune().nopwr && (pl.pwx == 1 || tune().pwrall) && pl.co_tiles == 1 && pwr_lds_bytes(pl.pwx, pl.pwx_steps) <= 160 * 1024 &&
        pl.pwx_steps >= 2 && c.Cin == 16 * pl.pwx_steps && c.Win % 8 == 0) {
        const int tiles = cdiv(a.TGp, 4);                            // 32 pixels x all output channels per wave
        // persistent workgroups of four waves: as many per CU as LDS and registers allow (16 accumulator tiles fill a
        // SIMD's register file, 8 leave room for a second wave, 4 for a third)
        const size_t lds = pwr_lds_bytes(pl.pwx, pl.pwx_steps);
        int per_cu = std::min((int)(160 * 1024 / lds), pl.pwx == 4 ? 1 : pl.pwx == 2 ? 2 : 3);
        if (tune().wgs > 0) per_cu = std::min(per_cu, tune().wgs);
        const int wgs = std::min(per_cu * dev->cu_count, cdiv(tiles, 4));
        const int waves = 4 * wgs, rem = tiles % waves;
        a.items = a.items_whole = tiles;
        // a last round that not every wave takes part in is cut into sub-tiles of 32 output channels where that
        // makes it shorter
        if (rem > 0 && pl.pwx > 1 && cdiv(rem * pl.pwx, waves) < pl.pwx && !tune().nohalf) {
            a.items_whole = tiles - rem;
            a.items = a.items_whole + rem * pl.pwx;
        }
        int prc;
        {
            KernelTimer timer(st);
            prc = launch_pwr_f16(pl.pwx, a, wgs, st);
        }
        if (prc != 0) return PHX_ERR_NOT_SUPPORTED;
        PHX_HIP(hipGetLastError());
        snprintf(g_name_buf, sizeof(g_name_buf), "%sqconv_%s_f16mfmapwr_p16_f16_wco%d_k%d_wgs%d_sub%d%s", g_name_prefix,
                 map == MAP_FWD ? "fwd" : "dgrad", pl.pwx, pl.pwx_steps, wgs, a.items - a.items_whole, a.addend ? "_add" : "");
        label_groups(gb.n);
        g_last_kernel = g_name_buf;
        say(p, map == MAP_FWD ? "forward" : "input gradient");
        return PHX_OK;
    }
    const int groups_per_tile = 8 * (4 / pl.pwx);
    const int whole = cdiv(a.TGp, groups_per_tile) * pl.co_tiles;
    const int slots = 2 * dev->cu_count;  // persistent workgroups, two per CU
    int blocks = std::min(whole, slots);
    a.items = a.items_whole = whole;
    // A last round that keeps at most half of the workgroups busy runs as half items (one of a wave's two column
    // tiles each): it then costs half an item's time.  With 1568 items on 512 workgroups that is 3.5 rounds for 4.
    const int rem = whole % blocks;
    if (!tune().nohalf) {
        if (2 * whole <= slots) { a.items_whole = 0; a.items = blocks = 2 * whole; }
        else if (rem > 0 && 2 * rem <= blocks) { a.items_whole = whole - rem; a.items = whole + rem; }
    }
    int rc;
    {
        KernelTimer timer(st);
        rc = launch_pwx_f16(pl.pwx, a, blocks, st);
    }
    if (rc != 0) return PHX_ERR_NOT_SUPPORTED;
    PHX_HIP(hipGetLastError());
    snprintf(g_name_buf, sizeof(g_name_buf), "%sqconv_%s_f16mfmapwx_p16_f16_wco%d_px%d_k%d_wgs%d_half%d%s", g_name_prefix,
             map == MAP_FWD ? "fwd" : "dgrad", pl.pwx, 64 * (4 / pl.pwx), pl.pwx_steps, blocks, a.items - a.items_whole,
             a.addend ? "_add" : "");
    label_groups(gb.n);
    g_last_kernel = g_name_buf;
    say(p, map == MAP_FWD ? "forward" : "input gradient");
    return PHX_OK;
}

// Channels-last pointwise convolutions on fp16 matrix cores run natively on the channels-last form of that kernel
// (forward and input gradient; the filter gradient and every other channels-last call go through the transposes
// of ChannelsLast below).
static int pwx_wco(int cout) {
    if (tune().tile_wco == 1 || tune().tile_wco == 2 || tune().tile_wco == 4) return tune().tile_wco;
    return cout > 64 ? 4 : cout > 32 ? 2 : 1;
}

// The channels-last kernel reads a K step as 32 bytes of every pixel's channel vector, so the steps of a work item
// come back to the same cache lines; with one output sub-tile the item is 256 pixels wide and the items in flight
// on an XCD hold more lines than its L2 keeps (64 -> 16 channels at 56x56, N=64: 78 us, where 16 -> 64 takes 25).
// From two K steps on, narrow outputs take the 128-pixel item of two sub-tiles, half of it empty rows: 39 us.
static int pwx_wco_nhwc(int cin, int cout) {
    const int wco = pwx_wco(cout);
    return (wco == 1 && cin > 16 && !tune().tile_wco) ? 2 : wco;
}

static bool nhwc_native(const Problem& p, int pass) {
    return p.nhwc && (pass == PHX_PASS_FWD || pass == PHX_PASS_BWD_DATA) && is_pointwise_unit(p) && !is_empty(p) &&
           use_f16_mfma(p, pass) && !p.real_input && p.groups == 1 && p.ci % 8 == 0 && p.co % 8 == 0 &&
           (long)p.n * p.h * p.w < (1L << 30) && !tune().nopwx;
}

// Reduction slices of a channels-last pointwise pass (see corr_slices for the idea): few work items and a long
// reduction -- Dense layers on a few hundred rows, deep pointwise layers on small batches -- run as Z slices of the
// reduced channels in one launch and a pass that adds the partial tensors.  Z = the largest power of two that keeps at
// least 32 channels (a multiple of 16) and 8 steps of 16 channels per slice and at most one item per CU; at least 4.
static int nhwc_slices(const Problem& p, int map) {
    if (tune().kslices == 0) return 0;
    const int cin = map == MAP_FWD ? p.ci : p.co, cout = map == MAP_FWD ? p.co : p.ci;
    const auto fits = [&](int z) { return cin % z == 0 && (cin / z) % 16 == 0 && cin / z >= 32; };
    if (tune().kslices > 1) return fits(tune().kslices) ? tune().kslices : 0;
    const int wco = pwx_wco_nhwc(cin, cout);
    const long items = (long)cdiv((int)((long)p.n * p.h * p.w), 64 * (4 / wco)) * cdiv(cout, 32 * wco);
    const int steps = cdiv(cin, 16);
    int Z = 1;
    while (fits(2 * Z) && items * 2 * Z <= 256 && steps / (2 * Z) >= 8) Z *= 2;
    return Z >= 4 ? Z : 0;
}

static size_t nhwc_native_workspace(const Problem& p, int pass) {
    const int map = pass == PHX_PASS_FWD ? MAP_FWD : MAP_DGRAD;
    const int cin = pass == PHX_PASS_FWD ? p.ci : p.co, cout = pass == PHX_PASS_FWD ? p.co : p.ci;
    const int wco = pwx_wco_nhwc(cin, cout);
    if (const int Z = nhwc_slices(p, map))  // Z partial result tensors, then Z packed images
        return align_up((size_t)Z * 4 * p.n * p.h * p.w * cout * 2, 256) +
               (size_t)Z * align_up(pwx_packed_bytes(wco, cdiv(cout, 32 * wco), cdiv(cin / Z, 16)), 256);
    return align_up(pwx_packed_bytes(wco, cdiv(cout, 32 * wco), cdiv(cin, 16)), 256);
}

static int run_pwx_nhwc(const Problem& p, int map, hipStream_t st, const void* in, const void* w, const void* bias, void* out,
                        void* ws, size_t ws_bytes) {
    const bool dry = g_pack.dry();
    if (!dry && (!in || !w || !out)) return PHX_ERR_INVALID_ARGUMENT;
    const int Z = nhwc_slices(p, map), slices = Z ? Z : 1;
    const int cin_all = map == MAP_FWD ? p.ci : p.co, cin = cin_all / slices, cout = map == MAP_FWD ? p.co : p.ci;
    const int wco = pwx_wco_nhwc(cin_all, cout), co_tiles = cdiv(cout, 32 * wco), nsteps = cdiv(cin, 16);
    const long np = (long)p.n * p.h * p.w;
    // sliced: the partial tensors lie at the front of the workspace, the packed images of the slices behind them
    const long count = 4L * np * cout;
    const size_t partial_bytes = Z ? align_up((size_t)Z * count * 2, 256) : 0;
    char* partial = static_cast<char*>(ws);
    if (Z && !dry) {
        if (ws_bytes < partial_bytes || !ws) return PHX_ERR_WORKSPACE;
        ws = partial + partial_bytes; ws_bytes -= partial_bytes;
    }
    const size_t image = align_up(pwx_packed_bytes(wco, co_tiles, nsteps), 256);
    const PackSlot slot = pack_slot(ws, ws_bytes, Z ? image * Z : pwx_packed_bytes(wco, co_tiles, nsteps));
    if (slot.rc != PHX_OK) return slot.rc;
    ws = slot.dst;
    // bytes from a slice's reduced channels to the next slice's in the filter: input channels forward, output channels backward
    const long w_step = (long)cin * (map == MAP_FWD ? p.fs.si : p.fs.so) * 2;
    PackArgs pa{};
    pa.groups = slices; pa.g_w = w_step; pa.g_out = (long)image;
    pa.w = w; pa.out = ws;
    pa.wcs = p.fs.wcs; pa.so = p.fs.so; pa.si = p.fs.si; pa.skh = p.fs.skh; pa.skw = p.fs.skw;
    pa.Co = map == MAP_FWD ? p.co : cin; pa.Ci = map == MAP_FWD ? cin : p.ci; pa.Kh = 1; pa.Kw = 1; pa.khm = 0; pa.khs = 1; pa.kwm = 0; pa.kws = 1;
    pa.rows = cout; pa.red = cin; pa.row_tiles = co_tiles; pa.nchunks = nsteps;
    if (slot.pack_now && launch_pack_filters_pwx(map, wco, nsteps, pa, st) != 0) return PHX_ERR_NOT_SUPPORTED;
    for (int z = 0; z < slices; ++z) {  // (the combined packing launch takes one job per image)
        PackArgs one = pa;
        one.groups = 1;
        one.w = at_bytes(pa.w, z * w_step);
        one.out = at_bytes(pa.out, z * image);
        if (const int rrc = record_pwx_job(one, map, wco, nsteps)) return rrc;
    }
    if (!slot.compute) return PHX_OK;
    DeviceState* dev = nullptr;
    if (const int rc = device_state(&dev)) return rc;
    PwxArgs a{};
    a.in = static_cast<const _Float16*>(in); a.in_cs = np * cin_all;
    a.wpk = static_cast<const f16x8*>(ws); a.bias = Z ? nullptr : static_cast<const _Float16*>(bias);
    a.out = Z ? reinterpret_cast<_Float16*>(partial) : static_cast<_Float16*>(out); a.out_cs = np * cout;
    a.N = p.n; a.Cin = cin; a.CinS = cin_all; a.Cout = cout; a.CoutS = cout; a.HW = p.h * p.w; a.NP = (int)np;
    a.co_tiles = co_tiles; a.nsteps = nsteps;
    a.items = cdiv((int)np, 64 * (4 / wco)) * co_tiles;
    a.groups = slices; a.g_in = (long)cin * 2; a.g_w = (long)image; a.g_bias = 0; a.g_out = count * 2;
    const int blocks = std::min(a.items, 2 * dev->cu_count);
    int rc;
    {
        KernelTimer timer(st);
        rc = launch_pwx_nhwc_f16(wco, a, blocks, st);
    }
    if (rc != 0) return PHX_ERR_NOT_SUPPORTED;
    PHX_HIP(hipGetLastError());
    if (Z) {
        const bool add = map == MAP_DGRAD && g_addend.dx == out && g_addend.ptr && !g_addend.fused;
        launch_slice_sum(true, partial, Z, count, out, bias, add ? g_addend.ptr : nullptr, 1, cout, count / 4, st);
        PHX_HIP(hipGetLastError());
        if (add) g_addend.fused = true;
    }
    snprintf(g_name_buf, sizeof(g_name_buf), "qconv_%s_f16mfmapwxcl_p16_f16_wco%d_px%d_k%d_wgs%d", map == MAP_FWD ? "fwd" : "dgrad",
             wco, 64 * (4 / wco), nsteps, blocks);
    if (Z) snprintf(g_name_buf + strlen(g_name_buf), sizeof(g_name_buf) - strlen(g_name_buf), "_kslices%d", Z);
    g_last_kernel = g_name_buf;
    say(p, map == MAP_FWD ? "forward (channels-last)" : "input gradient (channels-last)");
    return PHX_OK;
}

static int run_corr(const Problem& p, const Corr& creal, int map, hipStream_t st, const void* in, const void* w,
                    const void* bias, void* out, void* ws, size_t ws_bytes) {
    const bool f16 = use_f16_mfma(p, map == MAP_FWD ? PHX_PASS_FWD : PHX_PASS_BWD_DATA);
    int pw = 0;
    Corr c;
    FwdPlan pl;
    if (!plan_corr(creal, p.mode, f16, c, pl, pw)) return PHX_ERR_NOT_SUPPORTED;
    if (pl.pwx) return run_pwx(p, creal, pl, map, st, in, w, bias, out, ws, ws_bytes);
    const GroupBatch gb = g_batch;
    const size_t image = align_up(pl.wpk_bytes, 256);  // (group after group where one launch runs them all)
    const PackSlot slot = pack_slot(ws, ws_bytes, gb.n > 1 ? image * gb.n : pl.wpk_bytes);
    if (slot.rc != PHX_OK) return slot.rc;
    ws = slot.dst;

    FwdVariant v;
    v.half_storage = p.dtype == PHX_F16; v.f16_mfma = f16; v.mode = pl.kmode; v.map = map;
    v.WCO = pl.WCO; v.NTW = pl.NTW; v.CK = pl.CK; v.P2LOG = pl.P2LOG; v.wgs = pl.wgs; v.lds_bytes = pl.lds_bytes;
    v.lds_filters = pl.lds_filters; v.ngroups = pl.ngroups; v.pairs = pl.pairs; v.chunks = pl.chunks; v.pw = pw; v.vstage = pl.vstage;

    PackArgs pa{};
    pa.groups = gb.n; pa.g_w = (long)gb.w; pa.g_out = (long)image;
    pa.w = w; pa.out = ws;
    pa.wcs = p.fs.wcs; pa.so = p.fs.so; pa.si = p.fs.si; pa.skh = p.fs.skh; pa.skw = p.fs.skw;
    pa.Co = p.co; pa.Ci = p.ci; pa.Kh = creal.Kh; pa.Kw = creal.Kw;
    pa.khm = creal.khm; pa.khs = creal.khs; pa.kwm = creal.kwm; pa.kws = creal.kws;
    pa.rows = c.Cout; pa.red = creal.Cin; pa.row_tiles = pl.co_tiles * pl.WCO;
    pa.nchunks = f16 ? pl.nchunks : pl.nchunks * (pl.CK / F32_CK);
    // (LDS images: one thread per packed half, in 8-product form one thread per element of eight lane vectors)
    const long pack_items = pl.lds_filters ? (long)(pl.wpk_bytes / 2) / (pl.kmode == 8 ? 8 : 1)
                                            : (long)pa.row_tiles * pa.nchunks * creal.Kh * creal.Kw * (f16 ? 1 : 4) * 64;
    if (pl.lds_filters) pa.row_tiles = pl.co_tiles;  // packed per workgroup tile of WCO*32 channels
    const int pack_blocks = (int)std::min<long>((pack_items + WG_THREADS - 1) / WG_THREADS, 4096);

    ConvArgs a{};
    a.groups = gb.n; a.g_in = (long)(map == MAP_FWD ? gb.x : gb.y); a.g_w = (long)image; a.g_bias = (long)gb.b;
    a.g_out = (long)(map == MAP_FWD ? gb.y : gb.x);
    // channels per image in memory on the input and output side of this correlation (grouped convolutions: slices)
    const int cin_mem = (map == MAP_FWD) ? p.ci_mem : p.co_mem, cout_mem = (map == MAP_FWD) ? p.co_mem : p.ci_mem;
    a.in.base = in; a.in.comp_stride = (long)c.N * cin_mem * c.Hin * c.Win; a.in.Cs = cin_mem;
    a.in.N = c.N; a.in.C = creal.Cin; a.in.Hd = c.Hin; a.in.Wd = c.Win; a.in.uh = c.uh; a.in.uw = c.uw; a.in.pw = pw; a.in.tall = pl.tall;
    // channels-last tensors on both sides: only the chunk-staging fp16 kernel reads them (nhwc_window_native holds)
    const bool cl = g_window_cl;
    if (cl && !(f16 && pl.lds_filters && pl.chunks && !pw)) return PHX_ERR_RUNTIME;
    a.in.nhwc = cl; a.nhwc = cl;
    // real-valued input: the forward pass reads one component, the others are zero
    a.in.ncomp = (p.real_input && map == MAP_FWD) ? 1 : 4;
    a.wpk = ws; a.bias = bias; a.out = out;
    a.out_cs = (long)c.N * cout_mem * c.Hout * c.Wout;
    a.Cout = c.Cout; a.CoutS = cout_mem; a.Hout = c.Hout; a.Wout = c.Wout;
    a.taps = c.Kh * c.Kw; a.Kw = c.Kw; a.dh = c.dh; a.dw = c.dw; a.sh = c.sh; a.sw = c.sw; a.pt = c.pt; a.pl = c.pl;
    a.NB = pl.NB; a.TH = pl.TH; a.TW = pl.TW; a.HTH = pl.HTH; a.HTW = pl.HTW; a.HP = pl.HP; a.HPp = pl.HPp;
    a.tiles_n = pl.tiles_n; a.tiles_h = pl.tiles_h; a.tiles_w = pl.tiles_w; a.co_tiles = pl.co_tiles;
    a.nchunks = pl.nchunks;
    // pixels a lane may store as one word: the groups must not straddle tile rows or the image edge
    a.vec = (pl.TW % 4 == 0 && c.Wout % 4 == 0) ? 4 : (pl.TW % 2 == 0 && c.Wout % 2 == 0) ? 2 : 1;
    if (tune().vec > 0) a.vec = std::min(a.vec, tune().vec);

    int rc = 0;
    if (slot.pack_now) rc = f16 ? launch_pack_filters_f16(v, pa, pack_blocks, st) : launch_pack_filters(v, pa, pack_blocks, st);
    if (rc != 0) return PHX_ERR_NOT_SUPPORTED;
    if (g_pack.mode == PackSession::RECORD) {
        for (int g = 0; g < gb.n; ++g) {  // (the combined packing launch takes one job per image)
            PackJob j{};
            j.a = pa; j.a.groups = 1;
            j.a.w = at_bytes(pa.w, g * gb.w);
            j.a.out = at_bytes(pa.out, g * image);
            j.kind = !f16 ? PACK_F32 : pl.lds_filters ? PACK_F16_LDS : PACK_F16;
            j.half_storage = v.half_storage; j.mode = pl.kmode; j.map = map; j.WCO = pl.WCO; j.ngroups = pl.ngroups; j.pw = pw;
            if (const int rrc = record_pack_job(j, pack_items)) return rrc;
        }
    }
    if (!slot.compute) return PHX_OK;
    {
        KernelTimer timer(st);
        rc = f16 ? launch_fwd_f16(v, a, st) : launch_fwd_f32(v, a, st);
    }
    if (rc != 0) return PHX_ERR_NOT_SUPPORTED;
    PHX_HIP(hipGetLastError());
    snprintf(g_name_buf, sizeof(g_name_buf), "%sqconv_%s_%smfma%s%s_p%d_%s_wco%d_ntw%d_ck%d_%s%dx%dx%d", g_name_prefix,
             map == MAP_FWD ? "fwd" : "dgrad", f16 ? "f16" : "f32", pl.lds_filters ? (pw ? "ldspw" : pl.chunks ? "ldsc" : "lds") : "",
             cl ? "cl" : "", pl.kmode, p.dtype == PHX_F32 ? "f32" : "f16", pl.WCO, pl.NTW, pl.CK, pl.tall ? "flat" : "tile", pl.NB, pl.TH, pl.TW);
    label_groups(gb.n);
    g_last_kernel = g_name_buf;
    say(p, map == MAP_FWD ? "forward" : "input gradient");
    return PHX_OK;
}

// -------------------------------------------------------------------------------------------
// Filter gradient
// -------------------------------------------------------------------------------------------
struct WgPlan {
    int TPW, NB, TH, TW, KP, KPp, HPp, HPx, HTH, HTWmax;
    int tiles_n, tiles_h, tiles_w, co_tiles, ci_tiles, CoP, CiP, groups_per_row, Z;
    int MT, NT;  // fp16 kernel: 32*MT x 32*NT channel tile
    int kmode;   // product formulation the kernel runs in (see wgrad_f16_formulation, wgrad_f32_formulation)
    bool vec;    // fp32 kernel: windows staged as groups of 4 positions
    int ksets;   // fp32 kernel: wave sets per workgroup, each with a reduction slice of its own
    int SW, cpr, nchunks, ntiles;  // fp16 kernel: stride along W, 8-pixel chunks per output row / in total, pixel tiles
    bool flat;   // fp16 kernel: the chunk list runs over whole image planes (cpr = chunks per plane)
    bool realx;  // real-valued input, few channels: the one-product kernel of phx_kernels_realx.h
    int rows_per_wg, pitch;  // ... its output rows per workgroup (Z workgroups) and LDS row pitch; ntiles = column tiles
    size_t lds_bytes, partial_bytes;
};

// Reduction slices of a filter gradient on the fp32 matrix cores.  xy workgroups share a slice (channel tiles x tap groups), a slice walks
// ceil(ntiles / Z) pixel tiles, `slots` workgroups run at a time.  With few workgroups per slice one round of
// workgroups is best (Z = slots / xy: small partial sums, no straggler round) and is kept wherever it fills four
// fifths of the slots; where xy alone is a good part of a round (large channel counts: 256 -> 256, 3x3, one tap per
// workgroup = 144) it leaves CUs idle, and several rounds of shorter workgroups fill them.  The cost below is in units of one pixel tile of one workgroup: rounds x
// (tiles per workgroup + one tile's worth of start-up and epilogue) + slices x the time to write and read back a
// slice of partial sums (slice_bytes twice at 5 TB/s, against tile_flops at the 0.45 TFLOP/s one CU sustains).
// (The fp16 kernels keep the one-round rule: two of their workgroups share a CU, which this count of rounds does
// not describe -- tried there, it cost the small layers of a ResNet 10-35 %.)
static int reduction_slices(int xy, int ntiles, int slots, double slice_bytes, double tile_flops) {
    xy = std::max(1, xy);
    const int one_round = std::max(1, std::min(ntiles, slots / xy));
    if ((double)xy * one_round >= 0.8 * slots) return one_round;
    const double tile_seconds = tile_flops / 0.45e12;
    const double slice_cost = (2.0 * slice_bytes / 5e12) / tile_seconds;
    const int zmax = std::max(1, std::min(ntiles, std::max(slots / xy, 32)));
    int best_z = 1;
    double best_cost = 1e300;
    for (int z = 1; z <= zmax; ++z) {
        const long rounds = ((long)xy * z + slots - 1) / slots;
        const double cost = (double)rounds * ((ntiles + z - 1) / z + 1.0) + slice_cost * z;
        if (cost < best_cost) { best_cost = cost; best_z = z; }
    }
    return best_z;
}

static bool group_batchable(const Problem& p, int pass);

// the groups that share the GPU with one group's filter-gradient launch: its reduction slices fill that share
static int wgrad_group_share(const Problem& p) { return group_batchable(p, PHX_PASS_BWD_WEIGHTS) ? p.groups : 1; }

static void finish_wgrad_plan(const Problem& p, int CoT, int CiT, int per_cu, WgPlan& best) {
    best.co_tiles = cdiv(p.co, CoT); best.ci_tiles = cdiv(p.ci, CiT);
    best.CoP = best.co_tiles * CoT; best.CiP = best.ci_tiles * CiT;
    best.groups_per_row = cdiv(p.kw, best.TPW);
    const int xy = best.co_tiles * best.ci_tiles * best.groups_per_row * p.kh;
    const int ntiles = best.tiles_n * best.tiles_h * best.tiles_w;
    int target = std::max(1, 256 * per_cu / wgrad_group_share(p));  // one round of workgroups
    if (tune().wgs > 0) target = tune().wgs;
    const double slice_bytes = (double)std::max(1, best.ksets) * p.kh * p.kw * 4 * best.CoP * best.CiP * sizeof(float);
    const double tile_flops = 2.0 * best.KP * CoT * CiT * best.kmode * std::min(best.TPW, p.kw);
    best.Z = tune().oldplan ? std::max(1, std::min(ntiles, target / std::max(1, xy)))
                            : reduction_slices(xy, ntiles, target, slice_bytes, tile_flops);
    best.partial_bytes = (size_t)best.Z * p.kh * p.kw * 4 * best.CoP * best.CiP * sizeof(float);
}

// The fp32-MFMA filter gradient runs in the product mode that was asked for.  In 8-product mode every tap has a
// workgroup of its own (its 8 accumulator sets leave no room for more), so the taps of a filter row each stage the
// same gradient tile, where the 16-product kernel shares it between three taps; with reduction slices that fill the
// CUs (reduction_slices) and row-pair tiles of 32 positions the halved multiplications still win on the smallest
// images (fp16 tensors under the backward32 policy, 3x3, 256 -> 256 @ 14x14: 3.2 ms factorized against 5.1 ms).
// PHX_TUNE_OLDPLAN brings back the earlier choice (16-product kernel for rows of at most 20 positions).
static int wgrad_f32_formulation(const Problem& p) {
    return (p.mode == 8 && p.kw % 3 == 0 && p.wo <= 20 && !tune().wg8 && tune().oldplan) ? 16 : p.mode;
}

// fp32-MFMA kernel: 64x64 channel tiles, pixel tile and input window of at most 32 positions
static bool plan_wgrad_f32(const Problem& p, WgPlan& best) {
    best.kmode = wgrad_f32_formulation(p);
    const int TPW = (best.kmode == 16) ? 3 : 1;
    const int nkw = std::min(TPW, p.kw);
    double best_score = -1.0;
    const bool small_image = p.ho * p.wo < 100;
    for (int vec = 0; vec < 2; ++vec) {  // vec: windows staged as groups of 4 positions (16-byte loads)
        // KPp + HPp (+ offsets) per staged channel; the eight-wave workgroups have their CU, and its LDS, to themselves
        const int budget = (wgrad_f32_ksets(best.kmode, vec != 0) == 2 && !tune().oldplan ? 72 * 1024 / 4 : LDS_FLOATS_MAX) / (4 * 64);
        // (a vector tile may reach past the row end -- 16 columns for a row of 14 -- its last positions masked like
        // those of any edge tile: one long tile per row pair instead of two short ones)
        for (int TW = vec ? 4 : 1; TW <= std::min(vec && !tune().oldplan ? (p.wo + 3) & ~3 : p.wo, 64); TW += vec ? 4 : 1) {
            for (int TH = 1; TH <= p.ho; ++TH) {
                for (int NB = 1; NB <= p.n; ++NB) {
                    if (NB > 1 && !(TH == p.ho && TW == p.wo)) break;
                    const int pix = NB * TH * TW;
                    const int KP = (pix + 1) & ~1;
                    const int HTH = (TH - 1) * p.sh + 1;
                    int HTW = (TW - 1) * p.sw + (nkw - 1) * p.dw + 1;
                    if (vec) HTW = (HTW + 3) & ~3;
                    const int HPx = NB * HTH * HTW;
                    const int KPp = KP | 1, HPp = HPx | 1;  // odd pitches: bank-conflict-free 4-byte reads
                    if (pix > 32 || HPx > 32) break;
                    if (KPp + HPp + (KP + 255) / 256 > budget) break;
                    const int tn = cdiv(p.n, NB), th = cdiv(p.ho, TH), tw = cdiv(p.wo, TW);
                    const double eff = ((double)p.n * p.ho * p.wo) / ((double)tn * th * tw * KP);
                    // (a tile is a barrier pair and a staging round whatever its size: on 7x7 images four rows of 8 at 77 %
                    // fill beat one row of 8 at 88 % -- 512 channels, N=64: 2.46 against 4.32 ms, 128 channels 0.14 against
                    // 0.23 ms -- which the weight on the tile's positions expresses for images below 10x10)
                    const double score =
                        eff * (1.0 + (small_image ? tune().wg_kpw : 0.002) * KP) * (TW >= std::min(p.wo, 8) ? 1.0 : 0.5) * (vec ? 1.25 : 1.0);
                    if (score > best_score) {
                        best_score = score;
                        best.vec = vec != 0;
                        best.TPW = TPW; best.NB = NB; best.TH = TH; best.TW = TW; best.KP = KP; best.KPp = KPp;
                        best.HPp = HPp; best.HPx = HPx; best.HTH = HTH; best.HTWmax = HTW;
                        best.tiles_n = tn; best.tiles_h = th; best.tiles_w = tw;
                    }
                }
            }
        }
    }
    if (best_score < 0) return false;
    best.MT = best.NT = 2;
    best.ksets = wgrad_f32_ksets(best.kmode, best.vec);
    finish_wgrad_plan(p, 64, 64, best.ksets == 2 ? 1 : 2, best);  // (eight waves of 256 registers fill a CU)
    best.partial_bytes *= best.ksets;
    best.lds_bytes = ((size_t)4 * 64 * (best.KPp + best.HPp) + best.KP) * sizeof(float);
    return true;
}

// fp16-MFMA kernel: 32*MT x 32*NT channel tiles; reduction over 8-pixel chunks of the output rows, 8 chunks per tile
// On fp16 matrix cores the filter gradient is faster in its 16-product form whatever the product mode asks
// for: the factorized form halves the matrix instructions but must form lanes of BOTH operands with packed
// vector adds in front of every block (80 vector instructions per 8 MFMAs), and its eight accumulator sets
// leave no room to share a staged gradient tile between three taps (measured 128->128@28^2 3x3: 1016 against
// 794 TFLOP/s real-equivalent, pointwise 780 against 700).  UPSTRIDE_MEMORY_OPTIMIZED unset means "prefer
// speed" (src/backend/backend.hpp:36-66), so the 8-product mode runs this pass on the 16-product kernel;
// PHX_TUNE_WG8 keeps the factorized kernel (tests exercise it).
static int wgrad_f16_formulation(const Problem& p) {
    return (p.mode == 8 && !tune().wg8) ? 16 : p.mode;
}

// Real-valued input with few channels (the first layer of a network on images): one matrix product holds the whole
// filter gradient, see phx_kernels_realx.h.  q-ResNet-50 stem (7x7 stride 2 on 3 channels as 4x4 on 12 by
// space-to-depth, 16 output channels, N=64): 0.47 ms on the general kernel.
static bool plan_wgrad_realx(const Problem& p, WgPlan& best) {
    if (!p.real_input || p.dtype != PHX_F16 || channel_slices(p) || p.nhwc || tune().norealx) return false;
    if (p.sh != 1 || p.sw != 1 || p.dh != 1 || p.dw != 1 || p.kw > 4 || p.co > 16 || p.ci * p.kh * 4 > 192) return false;
    if (p.wo % 8 != 0 || p.w < 8 || p.pt < 0 || p.pl < 0 || p.pl > 7 || p.pr > 7) return false;
    const int cpr = p.wo / 8;
    if (4 * p.co * cpr > REALX_GI * WG_THREADS || p.ci * p.kw * cpr > REALX_XI * WG_THREADS) return false;
    if ((long)p.n * p.ci * p.h * p.w >= (1L << 31) || (long)p.n * p.co * p.ho * p.wo >= (1L << 31)) return false;
    best = WgPlan{};
    best.realx = true;
    best.kmode = 16;
    best.ntiles = cdiv(p.ci * p.kh * 4, 32);
    int pitch = (p.wo + 15) & ~15;
    while (pitch % 64 != 8) pitch += 8;
    best.pitch = pitch;
    best.lds_bytes = (size_t)(64 + 32 * best.ntiles) * pitch * 2;
    if (best.lds_bytes > 160 * 1024) return false;
    const int total_rows = p.n * p.ho;
    const int target = tune().wgs > 0 ? tune().wgs : 512;  // two workgroups per CU
    best.rows_per_wg = cdiv(total_rows, std::min(total_rows, target));
    best.Z = cdiv(total_rows, best.rows_per_wg);
    best.CoP = p.co; best.CiP = (p.ci + 3) & ~3;
    best.partial_bytes = (size_t)best.Z * p.kh * p.kw * 4 * best.CoP * best.CiP * sizeof(float);
    return true;
}

static bool plan_wgrad_f16(const Problem& p, WgPlan& best) {
    if (plan_wgrad_realx(p, best)) return true;
    best = WgPlan{};
    best.SW = p.sw;
    best.kmode = wgrad_f16_formulation(p);
    best.MT = p.co > 32 ? 2 : 1;
    best.NT = p.ci > 32 ? 2 : 1;
    if (tune().wg_mt > 0 && tune().wg_nt > 0) { best.MT = tune().wg_mt; best.NT = tune().wg_nt; }
    // taps of one filter row that share a workgroup (and with it the staged gradient tile): three, or four
    // where the row has a multiple of four taps and the channel tile leaves the registers for it
    const bool shifts = best.kmode == 16 && p.sw == 1 && p.dw == 1;
    best.TPW = (shifts && p.kw % 3 == 0) ? 3 : (shifts && p.kw % 4 == 0 && !(best.MT == 2 && best.NT == 2)) ? 4 : 1;
    auto lds_need = [&](int tpw) { return (size_t)(4 * 32 * best.MT + tpw * 4 * 32 * best.NT) * 72 * 2; };
    if (lds_need(best.TPW) > 160 * 1024) best.TPW = 1;  // (four shifted copies of a 64-channel input tile do not fit)
    if (tune().wg_tpw == 1) best.TPW = 1;
    const int CoT = 32 * best.MT, CiT = 32 * best.NT;
    // chunk list over whole planes where rows would leave their last chunk partly empty (see the kernel's header)
    best.flat = p.sh == 1 && p.sw == 1 && p.w == p.wo && p.h > 1 && p.wo >= 7 && p.wo % 8 != 0 && !tune().noflat;
    best.cpr = best.flat ? cdiv(p.ho * p.wo, 8) : cdiv(p.wo, 8);
    const long nchunks = (long)p.n * (best.flat ? 1 : p.ho) * best.cpr;
    if (nchunks > (1L << 28)) return false;
    best.nchunks = (int)nchunks;
    best.ntiles = cdiv(best.nchunks, 8);
    best.co_tiles = cdiv(p.co, CoT); best.ci_tiles = cdiv(p.ci, CiT);
    best.CoP = best.co_tiles * CoT; best.CiP = best.ci_tiles * CiT;
    best.groups_per_row = cdiv(p.kw, best.TPW);
    best.lds_bytes = (size_t)(4 * CoT + best.TPW * 4 * CiT) * 72 * 2;
    if (best.flat) {  // the kernel keeps the masks of a plane's chunks in LDS: small planes only (large ones waste little)
        const size_t tables = (size_t)(best.cpr + 1) * (best.TPW + 1) * 16 + (size_t)best.cpr * 8;
        if (best.lds_bytes + tables <= 160 * 1024) {
            best.lds_bytes += tables;
        } else {
            best.flat = false;
            best.cpr = cdiv(p.wo, 8);
            best.nchunks = (int)((long)p.n * p.ho * best.cpr);
            best.ntiles = cdiv(best.nchunks, 8);
        }
    }
    // one round of workgroups: as many reduction slices as fill every CU once (twice where two workgroups fit),
    // which keeps the partial sums small and lets no CU wait for a straggler round
    const int xy = best.co_tiles * best.ci_tiles * best.groups_per_row * p.kh;
    const int per_cu = best.lds_bytes <= 80 * 1024 ? 2 : 1;
    int target = std::max(1, 256 * per_cu / wgrad_group_share(p));
    if (tune().wgs > 0) target = tune().wgs;
    best.Z = std::max(1, std::min(best.ntiles, target / std::max(1, xy)));
    best.partial_bytes = (size_t)best.Z * p.kh * p.kw * 4 * best.CoP * best.CiP * sizeof(float);
    return true;
}

// strides along W other than 1 and 2 have no fp16-MFMA filter-gradient kernel: fp32 arithmetic serves them
static bool wgrad_on_f16_mfma(const Problem& p) {
    // the kernel addresses one component with 32-bit element offsets
    const long lim = (1L << 31) - 64;
    return use_f16_mfma(p, PHX_PASS_BWD_WEIGHTS) && (p.sw == 1 || p.sw == 2) && (long)p.n * p.ci_mem * p.h * p.w < lim &&
           (long)p.n * p.co_mem * p.ho * p.wo < lim;
}

static bool plan_wgrad(const Problem& p, bool f16mfma, WgPlan& best) {
    struct Entry { WgPlan pl; bool ok; };
    static PlanMemo<Entry> memo;
    // everything the two planners read
    const PlanKey key{{p.mode, p.n, p.ci, p.co, p.h, p.w, p.kh, p.kw, p.sh, p.sw, p.dh, p.dw, p.pt, p.pl, p.pb, p.pr,
                       p.ho, p.wo, (int)f16mfma, (int)p.real_input, (int)p.dtype, p.groups, (int)p.nhwc}};
    std::lock_guard<std::mutex> lock(g_plan_mutex);
    const Entry& hit = memo.get(key, [&] {
        Entry e{};
        e.ok = f16mfma ? plan_wgrad_f16(p, e.pl) : plan_wgrad_f32(p, e.pl);
        return e;
    });
    g_plan_memo_sizes[1] = (long)memo.size();
    best = hit.pl;
    return hit.ok;
}

static int run_wgrad(const Problem& p, hipStream_t st, const void* x, const void* g, void* dw, void* ws,
                     size_t ws_bytes) {
    const bool f16 = wgrad_on_f16_mfma(p);
    WgPlan pl;
    if (!plan_wgrad(p, f16, pl)) return PHX_ERR_NOT_SUPPORTED;
    const GroupBatch gb = g_batch;
    const size_t slab = align_up(pl.partial_bytes, 256);  // partial sums, group after group where one launch runs them all
    if (ws_bytes < (gb.n > 1 ? slab * gb.n : pl.partial_bytes) || !ws) return PHX_ERR_WORKSPACE;
    if (gb.n > 1 && f16 && pl.realx) return PHX_ERR_RUNTIME;  // (group_batchable keeps real-valued input out)
    if (f16 && pl.realx) {
        RealWgArgs ra{};
        ra.x = static_cast<const _Float16*>(x); ra.g = static_cast<const _Float16*>(g);
        ra.g_cs = (long)p.n * p.co * p.ho * p.wo;
        ra.partial = static_cast<float*>(ws);
        ra.N = p.n; ra.Ci = p.ci; ra.Co = p.co; ra.H = p.h; ra.W = p.w; ra.Ho = p.ho; ra.Wo = p.wo;
        ra.Kh = p.kh; ra.Kw = p.kw; ra.pt = p.pt; ra.pl = p.pl;
        ra.CoP = pl.CoP; ra.CiP = pl.CiP; ra.rows_per_wg = pl.rows_per_wg;
        ra.ncol = p.ci * p.kh * 4; ra.ntiles = pl.ntiles; ra.pitch = pl.pitch;
        {
            KernelTimer timer(st);
            if (launch_wgrad_f16_realx(ra, pl.Z, pl.lds_bytes, st) != 0) return PHX_ERR_RUNTIME;
        }
        PHX_HIP(hipGetLastError());
        ReduceArgs r{};
        r.partial = ra.partial; r.dw = dw;
        r.wcs = p.fs.wcs; r.so = p.fs.so; r.si = p.fs.si; r.skh = p.fs.skh; r.skw = p.fs.skw;
        r.Z = pl.Z; r.Co = p.co; r.Ci = p.ci; r.Kh = p.kh; r.Kw = p.kw; r.CoP = pl.CoP; r.CiP = pl.CiP;
        launch_reduce_wgrad(true, r, st);
        PHX_HIP(hipGetLastError());
        snprintf(g_name_buf, sizeof(g_name_buf), "%sqconv_wgrad_f16mfma_realx_f16_cols%d_rows%d_z%d", g_name_prefix, ra.ncol,
                 pl.rows_per_wg, pl.Z);
        say(p, "filter gradient (real-valued input)");
        return PHX_OK;
    }
    WgradArgs a{};
    a.groups = gb.n; a.g_x = (long)gb.x; a.g_g = (long)gb.y; a.g_partial = (long)slab;
    a.x.base = x; a.x.comp_stride = (long)p.n * p.ci_mem * p.h * p.w; a.x.N = p.n; a.x.C = p.ci; a.x.Cs = p.ci_mem; a.x.Hd = p.h; a.x.Wd = p.w;
    // channels-last tensors on both sides: only the 64x64-tile fp16 kernel stages them (nhwc_wgrad_native holds)
    const bool cl = g_window_cl;
    if (cl && !(f16 && pl.kmode == 16 && pl.MT == 2 && pl.NT == 2 && pl.SW == 1 && (pl.TPW == 1 || pl.TPW == 3))) return PHX_ERR_RUNTIME;
    a.x.uh = a.x.uw = 1; a.x.pw = 0; a.x.tall = 0; a.x.nhwc = cl; a.x.ncomp = p.real_input ? 1 : 4;
    a.g.base = g; a.g.comp_stride = (long)p.n * p.co_mem * p.ho * p.wo; a.g.N = p.n; a.g.C = p.co; a.g.Cs = p.co_mem; a.g.Hd = p.ho; a.g.Wd = p.wo;
    a.g.uh = a.g.uw = 1; a.g.pw = 0; a.g.tall = 0; a.g.nhwc = cl; a.g.ncomp = 4;
    a.partial = static_cast<float*>(ws);
    a.Kh = p.kh; a.Kw = p.kw; a.sh = p.sh; a.sw = p.sw; a.dh = p.dh; a.dw = p.dw; a.pt = p.pt; a.pl = p.pl;
    a.NB = pl.NB; a.TH = pl.TH; a.TW = pl.TW; a.KP = pl.KP; a.KPp = pl.KPp; a.HPp = pl.HPp; a.HTH = pl.HTH;
    a.HTWmax = pl.HTWmax; a.HPx = pl.HPx;
    a.tiles_n = pl.tiles_n; a.tiles_h = pl.tiles_h; a.tiles_w = pl.tiles_w;
    a.co_tiles = pl.co_tiles; a.ci_tiles = pl.ci_tiles; a.CoP = pl.CoP; a.CiP = pl.CiP;
    a.groups_per_row = pl.groups_per_row;
    a.cpr = pl.cpr; a.nchunks = pl.nchunks; a.ntiles = pl.ntiles; a.zsplit = pl.Z;
    a.flat = (f16 && pl.flat) ? 1 : 0; a.rows = a.flat ? 1 : p.ho;
    const int nblocks = pl.co_tiles * pl.ci_tiles * pl.groups_per_row * p.kh * pl.Z;
    const bool half_storage = p.dtype == PHX_F16;
    {
        KernelTimer timer(st);
        if (f16) {
            if ((cl ? launch_wgrad_f16_cl(pl.TPW, a, nblocks, pl.lds_bytes, st)
                    : launch_wgrad_f16(pl.kmode, pl.MT, pl.NT, pl.TPW, pl.SW, a, nblocks, pl.lds_bytes, st)) != 0)
                return PHX_ERR_RUNTIME;
        } else {
            launch_wgrad_f32(half_storage, pl.vec, pl.kmode, a, dim3(nblocks, grid_rows(gb.n)), pl.lds_bytes, st);
        }
    }
    PHX_HIP(hipGetLastError());
    ReduceArgs r{};
    r.groups = gb.n; r.g_partial = (long)slab; r.g_dw = (long)gb.w;
    r.partial = a.partial; r.dw = dw;
    r.wcs = p.fs.wcs; r.so = p.fs.so; r.si = p.fs.si; r.skh = p.fs.skh; r.skw = p.fs.skw;
    r.Z = f16 ? pl.Z : pl.Z * pl.ksets; r.Co = p.co; r.Ci = p.ci; r.Kh = p.kh; r.Kw = p.kw; r.CoP = pl.CoP; r.CiP = pl.CiP;
    launch_reduce_wgrad(half_storage, r, st);
    PHX_HIP(hipGetLastError());
    if (f16)
        snprintf(g_name_buf, sizeof(g_name_buf), "%sqconv_wgrad_f16mfma%s_p%d_f16_ch%dx%d_taps%d_sw%d%s_z%d", g_name_prefix, cl ? "cl" : "",
                 pl.kmode, 32 * pl.MT, 32 * pl.NT, pl.TPW, pl.SW, pl.flat ? "_flat" : "", pl.Z);
    else
        snprintf(g_name_buf, sizeof(g_name_buf), "%sqconv_wgrad_f32mfma%s_p%d_%s_tile%dx%dx%d_z%d", g_name_prefix, pl.vec ? "v" : "", pl.kmode,
                 p.dtype == PHX_F32 ? "f32" : "f16", pl.NB, pl.TH, pl.TW, pl.Z);
    label_groups(gb.n);
    g_last_kernel = g_name_buf;
    say(p, "filter gradient");
    return PHX_OK;
}

// Input gradient of a strided convolution by phases (see phase_merge_kernel): the rows h = sh*i + a of dx
// receive the filter rows kh with kh*dh = a + pt (mod sh), which form an arithmetic progression; row i of
// the phase reads gradient row i + (a + pt - kh*dh)/sh.  Per axis that is a unit-stride correlation with
// `taps` taps, dilation `dil` and `pad` rows of zero padding in front.
struct PhaseAxis {
    int taps, kmax, kstep, dil, pad, size;
};

static PhaseAxis phase_axis(int a, int extent, int k, int d, int s, int pad_before) {
    PhaseAxis ax{0, 0, 1, 1, 0, a < extent ? (extent - a + s - 1) / s : 0};
    int first = -1, second = -1;
    for (int kk = 0; kk < k; ++kk) {
        if ((a + pad_before - kk * d) % s != 0) continue;  // (C++ remainder: zero exactly for multiples, whatever the sign)
        if (first < 0) first = kk;
        else if (second < 0) second = kk;
        ax.kmax = kk;
        ++ax.taps;
    }
    if (ax.taps == 0) return ax;
    ax.kstep = second >= 0 ? second - first : 1;
    ax.dil = second >= 0 ? (ax.kstep * d) / s : 1;
    // tap u is filter tap kmax - u*kstep and reads gradient row i + off(kmax) + u*dil
    const int off_min = (a + pad_before - ax.kmax * d) / s;
    ax.pad = -off_min;
    return ax;
}

// Used for strided pointwise convolutions (one phase holds everything, the others are zero: 0.15 -> 0.08-0.11 ms
// on the downsampling layers of a ResNet).  With more than one tap the phases are several small launches
// each, and the zero-insertion form on the LDS kernel is the faster one at the sizes measured
// (3x3 stride 2, 32-128 channels: 0.08-0.11 ms against 0.13-0.19 ms); PHX_TUNE_PHASE=1 sends every strided
// input gradient through the phases, PHX_TUNE_PHASE=0 none.
constexpr int PHASES_MAX = 64;  // strides up to 8 x 8 (PhaseMergeArgs::off)
static bool dgrad_by_phases(const Problem& p) {
    if (p.banded) return false;
    if ((p.sh == 1 && p.sw == 1) || p.sh * p.sw > PHASES_MAX || is_empty(p) || channel_slices(p)) return false;
    if (tune().phase >= 0) return tune().phase != 0;
    if (p.kh == 1 && p.kw == 1) return true;
    // The largest windows (overlapping patch embeddings: 16x16 stride 8): the zero-inserted form stages the whole filter
    // window around every output position, and at the staging limit a tile is next to no outputs, while a phase has
    // ceil(k / s) taps per axis: 8 -> 32 channels at 64x64, N=2 4.65 ms against 1.09 ms for 64 launches of a 2x2 filter.
    // (Smaller windows keep the zero insertion at such sizes: 12x12 stride 6 0.34 against 0.59 ms, 11x11 stride 4 0.10
    // against 0.29 -- a phase is a packing and a convolution launch of some 8 us each.)
    if (((long)(p.kh - 1) * p.dh + 1) * ((((long)(p.kw - 1) * p.dw + 1) + 7) & ~7L) > 224) return true;
    // Large problems: zero insertion multiplies the arithmetic by sh * sw, which the launches of the phases cost less
    // than once there is enough of it and the phases' images are not tiny (fp16, N=64, 3x3 stride 2, zero insertion
    // against phases: 128 channels at 28x28 261 / 197 us, 256 at 28x28 967 / 509, 512 at 14x14 1064 / 611, 5x5 256 at
    // 28x28 2174 / 789; but 64 at 28x28 83 / 103, 128 at 14x14 78 / 153, 512 at 7x7 346 / 463)
    // In fp32 arithmetic the phases win at every size measured (N=64, 3x3: 16 channels at 56x56 359 / 125 us, 128 at
    // 14x14 622 / 353, 512 at 7x7 2967 / 1281, 256 at 28x28 10325 / 1809).
    if (!use_f16_mfma(p, PHX_PASS_BWD_DATA)) return true;
    const double flops = 32.0 * p.n * p.ci * p.co * p.ho * p.wo * p.kh * p.kw;
    return flops >= 40e9 && (long)p.h * p.w >= 196;
}

static Corr phase_corr(const Problem& p, const PhaseAxis& ah, const PhaseAxis& aw) {
    Corr c{p.n, p.co, p.ho, p.wo, p.ci, ah.size, aw.size, ah.taps, aw.taps, 1, 1, ah.dil, aw.dil, ah.pad, aw.pad, 1, 1,
           ah.kmax, ah.kstep, aw.kmax, aw.kstep};
    // a single tap over the whole gradient plane (strided pointwise convolutions): one long row per image
    if (ah.taps == 1 && aw.taps == 1 && !ah.pad && !aw.pad && ah.size == p.ho && aw.size == p.wo) {
        c.Win = p.ho * p.wo; c.Hin = 1; c.Wout = c.Win; c.Hout = 1;
    }
    c.ncomp = 4;
    return c;
}

static size_t workspace_plain(const Problem& p, int pass) {
    if (is_empty(p)) return 0;
    if (pass == PHX_PASS_BWD_WEIGHTS) {
        WgPlan pl;
        return plan_wgrad(flatten_pointwise(p), wgrad_on_f16_mfma(p), pl) ? align_up(pl.partial_bytes, 256) : 0;
    }
    int pw = 0;
    Corr c;
    FwdPlan pl;
    if (pass == PHX_PASS_BWD_DATA && dgrad_by_phases(p)) {
        // phase buffers (together the size of dx, each rounded up) + the largest packed sub-filter
        const size_t esize = p.dtype == PHX_F32 ? 4 : 2;
        size_t bufs = 0, wpk = 0;
        for (int a = 0; a < p.sh; ++a)
            for (int b = 0; b < p.sw; ++b) {
                const PhaseAxis ah = phase_axis(a, p.h, p.kh, p.dh, p.sh, p.pt), aw = phase_axis(b, p.w, p.kw, p.dw, p.sw, p.pl);
                if (!ah.taps || !aw.taps || !ah.size || !aw.size) continue;
                bufs += align_up((size_t)4 * p.n * p.ci * ah.size * aw.size * esize, 256);
                if (!plan_corr(phase_corr(p, ah, aw), p.mode, use_f16_mfma(p, pass), c, pl, pw)) return 0;
                wpk = std::max(wpk, align_up(pl.wpk_bytes, 256));
            }
        return bufs + wpk;
    }
    return plan_corr((pass == PHX_PASS_FWD) ? corr_forward(p) : corr_dgrad(p), p.mode, use_f16_mfma(p, pass), c, pl, pw)
               ? align_up(pl.wpk_bytes, 256)
               : 0;
}

// Space-to-depth view of a stride-2 convolution with at most 4 input channels (see phx_kernels_s2d.h):
// the unit-stride problem q on rearranged activations / filters, and the workspace the rearranged copies take.
struct S2dView {
    Problem q;
    S2dFilterArgs fa;
    size_t x2_bytes, w2_bytes;
};

static int floordiv(int a, int b) { return a >= 0 ? a / b : -((-a + b - 1) / b); }

static bool s2d_view(const Problem& p, S2dView& v) {
    if (p.banded) return false;
    if (p.sh != 2 || p.sw != 2 || p.dh != 1 || p.dw != 1 || p.ci > 4 || (p.kh < 3 && p.kw < 3) || is_empty(p)) return false;
    if (channel_slices(p)) return false;  // the rearranged copies are laid out for whole tensors
    if (tune().nos2d) return false;
    const int aminh = floordiv(-p.pt, 2), amaxh = floordiv(p.kh - 1 - p.pt, 2);
    const int aminw = floordiv(-p.pl, 2), amaxw = floordiv(p.kw - 1 - p.pl, 2);
    Problem& q = v.q;
    q = p;
    q.ci = 4 * p.ci; q.ci_mem = q.ci;
    q.h = (p.h + 1) / 2; q.w = (p.w + 1) / 2;
    q.kh = amaxh - aminh + 1; q.kw = amaxw - aminw + 1;
    q.sh = q.sw = 1;
    q.pt = -aminh; q.pl = -aminw;
    q.pb = p.ho - q.h - q.pt + q.kh - 1;
    q.pr = p.wo - q.w - q.pl + q.kw - 1;
    if (q.pb < 0 || q.pr < 0) return false;
    q.ho = out_size(q.h, q.kh, 1, 1, q.pt, q.pb);
    q.wo = out_size(q.w, q.kw, 1, 1, q.pl, q.pr);
    if (q.ho != p.ho || q.wo != p.wo) return false;
    const long taps2 = (long)q.kh * q.kw;
    q.fs.wcs = (long)q.co * q.ci * taps2; q.fs.so = q.ci * taps2; q.fs.si = taps2; q.fs.skh = q.kw; q.fs.skw = 1;
    const size_t esize = p.dtype == PHX_F32 ? 4 : 2;
    v.x2_bytes = align_up((size_t)(p.real_input ? 1 : 4) * p.n * q.ci * q.h * q.w * esize, 256);
    v.w2_bytes = align_up((size_t)4 * q.fs.wcs * esize, 256);
    S2dFilterArgs& f = v.fa;
    f.wcs = p.fs.wcs; f.so = p.fs.so; f.si = p.fs.si; f.skh = p.fs.skh; f.skw = p.fs.skw;
    f.Co = p.co; f.Ci = p.ci; f.Kh = p.kh; f.Kw = p.kw; f.K2h = q.kh; f.K2w = q.kw;
    f.pt = p.pt; f.pl = p.pl; f.aminh = aminh; f.aminw = aminw;
    return true;
}

// A strided, unpadded pointwise convolution as the unit-stride one on the rows and columns it reads (forward and
// filter gradient; the input gradient has its phases): the problem q on the subsampled input and that copy's size.
// q-ResNet-50's three downsampling shortcuts, N=64: forward 0.07 ms on the general kernel.
static bool subsample_view(const Problem& p, Problem& q, size_t& xs_bytes) {
    if (p.banded) return false;
    if (p.kh != 1 || p.kw != 1 || (p.sh == 1 && p.sw == 1) || p.pt || p.pl || p.pb || p.pr || is_empty(p)) return false;
    if (channel_slices(p) || p.nhwc || p.real_input || tune().nosub) return false;
    q = p;
    q.h = p.ho; q.w = p.wo; q.sh = q.sw = 1;
    if (out_size(q.h, 1, 1, 1, 0, 0) != p.ho || out_size(q.w, 1, 1, 1, 0, 0) != p.wo) return false;
    xs_bytes = align_up((size_t)4 * p.n * p.ci * p.ho * p.wo * (p.dtype == PHX_F32 ? 4 : 2), 256);
    return true;
}

static void subsample_input(const Problem& p, const void* x, void* xs, hipStream_t st) {
    SubsampleArgs a;
    a.src = x; a.dst = xs; a.planes = 4L * p.n * p.ci; a.H = p.h; a.W = p.w; a.H2 = p.ho; a.W2 = p.wo; a.sh = p.sh; a.sw = p.sw;
    launch_subsample(p.dtype == PHX_F16, a, st);
}

// the window of one output position -- ((kh-1) dh + 1) rows of ((kw-1) dw + 1) columns in whole 8-position chunks --
// exceeds what the matrix-core kernels stage (one position per thread)
static long window_positions(const Problem& p) { return ((long)(p.kh - 1) * p.dh + 1) * ((((long)(p.kw - 1) * p.dw + 1) + 7) & ~7L); }
static bool window_beyond_staging(const Problem& p) { return window_positions(p) > WG_THREADS; }

// Convolutions whose stride equals their filter extent (patch embeddings: 16x16 stride 16; 2x2 stride 2 and 4x4
// stride 4 downsampling), undilated, with no padding in front of the image: every input position belongs to one
// output position, so with the positions of a patch laid out as channels (patch_depth_kernel) the convolution is a
// POINTWISE one over ci * kh * kw channels on the ho x wo grid of patches -- all three passes, on the streaming
// kernels, where the windowed kernels spend a window's worth of staging per output position and the input gradient
// would multiply sh * sw - 1 inserted zeros for every value (16x16 stride 16 on 224x224 images: seconds).  The filter
// is used as it lies: its taps and input channels form one channel index with one stride -- (c, kh, kw) in OIHW,
// (kh, kw, c) in OHWI and HWIO -- and the filter gradient of the pointwise problem is written straight to it.
// One gather in front of the forward pass and the filter gradient, one scatter behind the input gradient.
struct PatchView {
    Problem q;
    int tap_major;
    size_t x_bytes;  // the input-side tensor as patches
};
static bool patch_view(const Problem& p, int pass, PatchView& v) {
    if (p.banded) return false;
    if (tune().nopatch || tune().direct || is_empty(p) || p.kh != p.sh || p.kw != p.sw || p.kh * p.kw == 1) return false;
    if (p.dh != 1 || p.dw != 1 || p.pt || p.pl || channel_slices(p) || g_window_cl) return false;
    // Patches of fewer than nine positions (2x2 stride 2): the windowed kernels' forward pass and fp16 filter gradient
    // beat a gather plus the pointwise kernels (N=64, fp16, windowed / patches, us: 24 -> 48 channels at 56x56 forward
    // 39 / 68, filter gradient 38 / 75; 128 -> 256 at 28x28 145 / 177, 118 / 190); the input gradient (zero insertion or
    // four phases against one pointwise pass and a scatter: 99 / 71, 102 / 53) and the filter gradient in fp32 arithmetic
    // (267 / 148) do not.  From 3x3 on every pass gains (4x4 stride 4, 32 -> 64 at 56x56: 45 / 141 / 258 -> 97 / 57 / 93).
    if (p.kh * p.kw < 9 && !tune().patchall &&
        (pass == PHX_PASS_FWD || (pass == PHX_PASS_BWD_WEIGHTS && use_f16_mfma(p, PHX_PASS_BWD_WEIGHTS) && wgrad_on_f16_mfma(p))))
        return false;
    const FilterStrides& f = p.fs;
    long si = 0;
    if (f.skh == p.kw * f.skw && f.si == (long)p.kh * p.kw * f.skw) { v.tap_major = 0; si = f.skw; }
    else if (f.skw == p.ci * f.si && f.skh == (long)p.kw * p.ci * f.si) { v.tap_major = 1; si = f.si; }
    else return false;
    if ((long)p.ci * p.kh * p.kw > (1L << 20)) return false;
    // the patch kernel's index arithmetic on one channel's image or patches is exact below that
    if ((long)p.h * p.w >= (1L << 24) || (long)p.kw * p.ho * p.wo >= (1L << 24)) return false;
    Problem& q = v.q;
    q = p;
    q.nhwc = false;  // (the patch tensor is channels-first)
    q.ci = q.ci_mem = p.ci * p.kh * p.kw;
    q.h = p.ho; q.w = p.wo; q.kh = q.kw = 1; q.sh = q.sw = 1; q.pt = q.pl = q.pb = q.pr = 0;
    q.fs.si = si; q.fs.skh = q.fs.skw = 0;
    v.x_bytes = align_up((size_t)(p.real_input ? 1 : 4) * p.n * q.ci * p.ho * p.wo * (p.dtype == PHX_F32 ? 4 : 2), 256);
    return true;
}
static void patch_depth(const Problem& p, const PatchView& v, const void* src, void* dst, bool to_caller, hipStream_t st) {
    PatchArgs a;
    a.src = src; a.dst = dst; a.rows = (p.real_input ? 1L : 4L) * p.n; a.C = p.ci; a.H = p.h; a.W = p.w; a.Ho = p.ho; a.Wo = p.wo;
    a.kh = p.kh; a.kw = p.kw; a.tap_major = v.tap_major;
    launch_patch_depth(p.dtype == PHX_F16, a, to_caller, st);
}

// Dilated convolutions beyond that limit (a 3x3 filter from dilation 8 on: the atrous pyramids of segmentation
// networks use 12, 18, 24, 36) with unit stride: an output position and every input position it reads lie whole
// dilations apart, so the convolution is dh x dw independent undilated convolutions on the phase images of its
// tensors (see dilation_phase_kernel; the input side counts its phases from pt % dh rows, pl % dw columns in front
// of the image, which leaves q whole rows and columns of padding).  They run as ONE undilated convolution q on a batch dh x dw
// times as long, between a pass that gathers the phase images of the input-side tensor and one that scatters the
// result's; the filter is used as it is, so the filter gradient comes out of q directly.  Phase images are padded
// with zeros to one size (rows beyond the image are what the padding behind it holds anyway); the padding behind
// the phase images is what gives q the output extent ceil(ho / dh) x ceil(wo / dw).
struct DilationView {
    Problem q;
    int Hp, Wp, Hop, Wop;      // extent of the input-side and output-side phase images
    size_t x_bytes, y_bytes;   // the two phase tensors
};
static bool dilation_view(const Problem& p, int pass, DilationView& v) {
    if (p.banded) return false;
    if (tune().nodilphase || tune().direct || is_empty(p) || (p.dh == 1 && p.dw == 1) || p.sh != 1 || p.sw != 1) return false;
    // (the filter gradient stages no halo window around its tiles: it takes the rewrite only where it has to)
    const long most = pass == PHX_PASS_BWD_WEIGHTS ? WG_THREADS : std::min<long>(tune().dilphase_min, WG_THREADS);
    // (channels-last calls: the rewrite works on the channels-first copies such a call goes through -- nhwc_window_native
    // and nhwc_wgrad_native leave these problems to the copies -- never on the caller's tensors)
    if (window_positions(p) <= most || channel_slices(p) || g_window_cl || p.real_input) return false;
    if ((long)p.n * p.dh * p.dw > (1L << 22)) return false;
    v.Hp = cdiv(p.h + p.pt % p.dh, p.dh); v.Wp = cdiv(p.w + p.pl % p.dw, p.dw); v.Hop = cdiv(p.ho, p.dh); v.Wop = cdiv(p.wo, p.dw);
    Problem& q = v.q;
    q = p;
    q.nhwc = false;  // (the phase tensors are channels-first)
    q.n = p.n * p.dh * p.dw; q.h = v.Hp; q.w = v.Wp; q.ho = v.Hop; q.wo = v.Wop; q.dh = q.dw = 1;
    q.pt = p.pt / p.dh; q.pl = p.pl / p.dw;
    q.pb = v.Hop + (p.kh - 1) - v.Hp - q.pt; q.pr = v.Wop + (p.kw - 1) - v.Wp - q.pl;
    if (q.pb < 0 || q.pr < 0 || window_beyond_staging(q)) return false;
    if (out_size(q.h, q.kh, 1, 1, q.pt, q.pb) != q.ho || out_size(q.w, q.kw, 1, 1, q.pl, q.pr) != q.wo) return false;
    // the phase kernels' index arithmetic on one channel's phase images is exact below that
    if ((long)v.Hp * v.Wp * p.dw >= (1L << 24) || (long)v.Hop * v.Wop * p.dw >= (1L << 24)) return false;
    const size_t esize = p.dtype == PHX_F32 ? 4 : 2;
    v.x_bytes = align_up((size_t)4 * q.n * p.ci * v.Hp * v.Wp * esize, 256);
    v.y_bytes = align_up((size_t)4 * q.n * p.co * v.Hop * v.Wop * esize, 256);
    return true;
}
// the phase images of the input-side (input = true) or output-side tensor of p, or the tensor back from them
static void dilation_phases(const Problem& p, const DilationView& v, bool input, const void* src, void* dst, bool to_caller, hipStream_t st) {
    DilationPhaseArgs a;
    a.src = src; a.dst = dst; a.rows = 4L * p.n; a.C = input ? p.ci : p.co; a.H = input ? p.h : p.ho; a.W = input ? p.w : p.wo;
    a.Hp = input ? v.Hp : v.Hop; a.Wp = input ? v.Wp : v.Wop; a.dh = p.dh; a.dw = p.dw;
    a.oh = input ? p.pt % p.dh : 0; a.ow = input ? p.pl % p.dw : 0;
    launch_dilation_phases(p.dtype == PHX_F16, a, to_caller, st);
}

// Filter gradient of a strided convolution by tap classes.  Along an axis the taps whose input rows kh * d - pt share
// a residue modulo the stride form an arithmetic progression k0, k0 + T, ... (T = s / gcd(s, d)), and for them
//   x[s * i + kh * d - pt] = xg[i + m * (T * d / s)],   xg[i] = x[s * i + k0 * d - pt]  (zero outside the image):
// a unit-stride, unpadded correlation of `taps` taps and dilation T * d / s on the gathered rows xg, of which
// out + (taps - 1) * dilation are read.  The filter gradient of class (ch, cw) is therefore a unit-stride filter
// gradient between xg and the output gradient, written to its own taps of dw through filter strides T times as
// long: the strided problem runs as (at most sh x sw) unit-stride ones on the fast kernels, each behind one gather.
// (3x3 stride 2: classes of 2x2, 2x1, 1x2 and 1x1 taps, nine taps' work in all.)
struct TapClass {
    int taps, k0, kstep, dil, origin, size;
};
static int tap_classes(int k, int d, int s, int pad_before, int out, TapClass* cls) {
    const int period = s / std::__gcd(s, d);
    int n = 0;
    for (int k0 = 0; k0 < std::min(k, period); ++k0) {
        TapClass c;
        c.k0 = k0; c.kstep = period; c.taps = (k - 1 - k0) / period + 1;
        c.dil = c.taps > 1 ? period * d / s : 1;
        c.origin = k0 * d - pad_before;
        c.size = out + (c.taps - 1) * c.dil;
        cls[n++] = c;
    }
    return n;
}
constexpr int TAP_CLASSES_MAX = 8;  // strides up to 8 along an axis

// Which strided filter gradients run that way: those that would otherwise fall to fp32 arithmetic although the
// policy allows fp16 matrix cores (strides beyond 2 along W have no fp16 kernel: 3x3 stride 3, 128 channels at
// 28x28, N=32 570 -> 204 us), and large ones, where the strided kernels' one tap per workgroup costs more than the
// gathers, the launches and the classes' own reductions.  3x3 stride 2, strided kernel against classes (us):
// fp16 matrix cores 512 channels at 28x28, N=32 1144 / 818, 512 at 14x14, N=64 772 / 521, 256 at 28x28 558 / 508, but
// 256 at 14x14 197 / 219, 128 at 28x28 139 / 229, 64 at 56x56 131 / 289; fp32 arithmetic 512 at 28x28 5708 / 3396,
// 512 at 14x14 4260 / 1973, 256 at 28x28 2169 / 1802, but 128 at 28x28 544 / 536, 64 at 28x28 151 / 223.
static bool wgrad_by_classes(const Problem& p) {
    if (p.banded) return false;
    if ((p.sh == 1 && p.sw == 1) || p.kh * p.kw == 1 || is_empty(p) || channel_slices(p) || p.real_input || g_window_cl) return false;
    if (p.sh > TAP_CLASSES_MAX || p.sw > TAP_CLASSES_MAX) return false;
    S2dView v;
    if (s2d_view(p, v)) return false;
    if (tune().wgphase >= 0) return tune().wgphase != 0;
    if (use_f16_mfma(p, PHX_PASS_BWD_WEIGHTS) && !wgrad_on_f16_mfma(p)) return true;
    const double flops = 32.0 * p.n * p.ci * p.co * p.ho * p.wo * p.kh * p.kw;
    return flops >= 200e9;
}

// the unit-stride problem of one class, its gathered input extent and the first tap's offset in the filter (elements)
static Problem wgrad_class_problem(const Problem& p, const TapClass& ch, const TapClass& cw, long& tap_offset) {
    Problem q = p;
    q.nhwc = false;
    q.h = ch.size; q.w = cw.size; q.kh = ch.taps; q.kw = cw.taps; q.sh = q.sw = 1; q.dh = ch.dil; q.dw = cw.dil;
    q.pt = q.pl = q.pb = q.pr = 0;
    q.fs.skh = p.fs.skh * ch.kstep; q.fs.skw = p.fs.skw * cw.kstep;
    tap_offset = ch.k0 * p.fs.skh + cw.k0 * p.fs.skw;
    return q;
}

// Tap bands.  The windowed kernels stage, for every output tile, the window of the WHOLE filter around it: at the
// staging limit (a 16x16 filter: 256 positions) a tile is a single output position and a pass takes 10-20 times what
// a 13x13 filter takes; beyond it nothing fits (vector-ALU kernels).  A convolution is the sum of the convolutions
// with the bands of its filter -- blocks of at most 8 window columns and 20 window rows, at most 160 positions --
// each an ordinary problem on the same tensors whose padding is the original one minus the band's offset (negative
// where the band starts inside the window), its filter the block's taps through the same strides.  Forward and
// input gradient run one pass per band into partial tensors and add them (slice_sum_kernel, with the bias); the
// filter gradient of a band IS that band's block of dw.  Used from 225 window positions on where no other rewrite
// (patches, dilation phases) applies; groups and real-valued input keep the vector-ALU kernels.
struct TapBand {
    int r0, rows, c0, cols;
};
constexpr int TAP_BANDS_MAX = 32;
static int tap_bands(const Problem& p, int pass, TapBand* bands) {
    if (p.banded || tune().nobands || tune().direct || is_empty(p) || channel_slices(p) || p.real_input || g_window_cl) return 0;
    if (window_positions(p) <= (pass == PHX_PASS_BWD_WEIGHTS ? WG_THREADS : 224)) return 0;
    // (a strided input gradient by phases has ceil(k / s) taps per axis and phase: small windows already; windows
    // beyond the staging limit do not get that far -- they would go to the vector-ALU kernels -- and take the bands)
    if (pass == PHX_PASS_BWD_DATA && !window_beyond_staging(p) && dgrad_by_phases(p)) return 0;
    const int bw = 7 / p.dw + 1, bh = 19 / p.dh + 1;  // ((bw-1) dw + 1 <= 8 columns, (bh-1) dh + 1 <= 20 rows
    const int nh = cdiv(p.kh, bh), nw = cdiv(p.kw, bw);
    if (nh * nw > TAP_BANDS_MAX || nh * nw < 2) return 0;
    int n = 0;
    for (int a = 0; a < nh; ++a)
        for (int b = 0; b < nw; ++b) {
            // (bands of even size: 16 columns as 8 + 8, 13 as 7 + 6)
            const int r0 = (int)((long)a * p.kh / nh), r1 = (int)((long)(a + 1) * p.kh / nh);
            const int c0 = (int)((long)b * p.kw / nw), c1 = (int)((long)(b + 1) * p.kw / nw);
            bands[n++] = TapBand{r0, r1 - r0, c0, c1 - c0};
        }
    return n;
}
static Problem band_problem(const Problem& p, const TapBand& t, long& tap_offset) {
    Problem q = p;
    q.banded = true;
    q.nhwc = false;
    q.has_bias = false;
    q.kh = t.rows; q.kw = t.cols;
    q.pt = p.pt - t.r0 * p.dh; q.pl = p.pl - t.c0 * p.dw;
    q.pb = p.pb - (p.kh - t.r0 - t.rows) * p.dh; q.pr = p.pr - (p.kw - t.c0 - t.cols) * p.dw;
    tap_offset = t.r0 * p.fs.skh + t.c0 * p.fs.skw;
    return q;
}

// Reduction slices of a forward / input-gradient pass.  Those kernels give a workgroup an output tile and the whole
// reduction over channels and taps, so a pass with few output tiles and many channels (small batches on deep
// layers: 512 channels at 7x7, N=1 is 16 workgroups of 288 steps) leaves most of the GPU idle however long it
// takes.  Such a pass runs as Z passes over Z slices of the reduced channels in ONE launch per kernel (the grid rows
// that run the groups of a grouped convolution: slice z reads its channels of the input-side tensor and of the
// filter and writes a partial result tensor of its own in the workspace), and a streaming kernel adds the partial
// tensors (and the bias) into the caller's tensor, in fp32 with one rounding.
// Z = the largest power of two that keeps at least 32 channels (a multiple of 16) and 8 reduction steps per slice
// and at most two workgroups per CU in flight; 0 = the pass runs unsliced (enough workgroups already; groups and
// real-valued input are never sliced).  The unit-stride problem on a subsampled copy (strided pointwise forward) and
// the phases of a strided input gradient are passes of their own and sliced as such (do_fwd, phase_slices).
static int slices_rule(const Problem& p, int pass, const Corr& creal) {
    Corr c;
    FwdPlan pl;
    int pw = 0;
    const bool f16 = use_f16_mfma(p, pass);
    if (!plan_corr(creal, p.mode, f16, c, pl, pw)) return 0;
    const int red = creal.Cin;
    const auto fits = [&](int z) { return red % z == 0 && (red / z) % 16 == 0 && red / z >= 32; };
    if (tune().kslices > 1) return fits(tune().kslices) ? tune().kslices : 0;
    const int cus = 256;  // (a constant, as in plan_forward: the workspace query answers without a device)
    // workgroups (items of the pointwise streaming kernel, which runs at most two per CU and needs longer slices) and
    // reduction steps of the unsliced pass
    const long wgs = pl.pwx ? (long)cdiv(creal.N * cdiv(creal.Hin * creal.Win, 8), 8 * (4 / pl.pwx)) * pl.co_tiles : pl.wgs;
    const long steps = pl.pwx ? pl.pwx_steps : (long)pl.nchunks * c.Kh * c.Kw;  // (c: a pointwise problem may run as a column of virtual taps)
    const long most = pl.pwx ? cus : 2L * cus;
    int Z = 1;
    while (fits(2 * Z) && wgs * 2 * Z <= most && steps / (2 * Z) >= 8) Z *= 2;
    // (on the fp16 matrix cores two slices pay for the extra pass over the result only where the unsliced pass leaves
    // half of the CUs without a workgroup: 64 -> 64 3x3 at 14x14, N=32, 128 workgroups 27 -> 23 us, at 56x56, N=1
    // 31 -> 24; but 256 -> 256 at 14x14, N=16, 256 workgroups 107 -> 115, 64 -> 64 at 56x56, N=4, 200 workgroups
    // 35 -> 43; in fp32 arithmetic they always do: 570 -> 410)
    if (f16 && !pl.pwx && Z == 2 && wgs <= cus / 2) return 2;
    return Z >= (f16 ? 4 : 2) ? Z : 0;
}

static bool nhwc_window_native(const Problem& p, int pass);
static int corr_slices(const Problem& p, int pass) {
    if (p.banded) return 0;
    if (tune().kslices == 0 || pass == PHX_PASS_BWD_WEIGHTS || is_empty(p)) return 0;
    if (channel_slices(p) || p.real_input || g_batch.n > 1 || g_window_cl) return 0;
    // (channels-last tensors: a call that goes through channels-first copies is sliced on those; one that runs on the
    // caller's tensors is not -- nhwc_window_native leaves the passes that would be sliced to the copies)
    if (p.nhwc && nhwc_window_native(p, pass)) return 0;
    if (pass == PHX_PASS_BWD_DATA && dgrad_by_phases(p)) return 0;  // (see phase_slices)
    if (pass == PHX_PASS_FWD) {
        S2dView v;
        Problem q;
        size_t xs_bytes = 0;
        if (s2d_view(p, v) || subsample_view(p, q, xs_bytes)) return 0;
    }
    return slices_rule(p, pass, pass == PHX_PASS_FWD ? corr_forward(p) : corr_dgrad(p));
}

// A strided input gradient that runs by phases (dgrad_by_phases): every phase is a pass of its own and is sliced like
// one, all by the Z that the rule gives for the phase with the most taps.
static int phase_slices(const Problem& p) {
    if (p.banded) return 0;
    if (tune().kslices == 0 || !dgrad_by_phases(p) || g_batch.n > 1 || g_window_cl) return 0;
    PhaseAxis bh{}, bw{};
    for (int a = 0; a < p.sh; ++a)
        for (int b = 0; b < p.sw; ++b) {
            const PhaseAxis ah = phase_axis(a, p.h, p.kh, p.dh, p.sh, p.pt), aw = phase_axis(b, p.w, p.kw, p.dw, p.sw, p.pl);
            if (!ah.taps || !aw.taps || !ah.size || !aw.size) continue;
            if (ah.taps * aw.taps > bh.taps * bw.taps) { bh = ah; bw = aw; }
        }
    return bh.taps * bw.taps ? slices_rule(p, PHX_PASS_BWD_DATA, phase_corr(p, bh, bw)) : 0;
}

// the problem of one slice, and the steps from a slice to the next in the tensors of the pass
struct SlicedCorr {
    Problem q;
    GroupBatch steps;
    size_t partial_bytes;  // Z partial result tensors
    long count;            // elements of one
    // (plane: positions per channel of the result tensor; 0 = the whole image, else those of one phase)
    SlicedCorr(const Problem& p, int pass, int Z, long plane = 0) : q(p) {
        const size_t esize = p.dtype == PHX_F32 ? 4 : 2;
        q.has_bias = false;
        steps.n = Z;
        if (pass == PHX_PASS_FWD) {
            q.ci = p.ci / Z;
            count = 4L * p.n * p.co * p.ho * p.wo;
            steps.x = (size_t)q.ci * p.h * p.w * esize;
            steps.y = (size_t)count * esize;
            steps.w = (size_t)q.ci * p.fs.si * esize;
        } else {
            q.co = p.co / Z;
            count = 4L * p.n * p.ci * (plane ? plane : (long)p.h * p.w);
            steps.y = (size_t)q.co * p.ho * p.wo * esize;
            steps.x = (size_t)count * esize;
            steps.w = (size_t)q.co * p.fs.so * esize;
        }
        partial_bytes = align_up((size_t)Z * count * esize, 256);
    }
};

static size_t workspace_for(const Problem& p, int pass) {
    PatchView patches;
    if (patch_view(p, pass, patches)) return patches.x_bytes + workspace_for(patches.q, pass);
    DilationView dilated;
    if (dilation_view(p, pass, dilated)) return dilated.x_bytes + dilated.y_bytes + workspace_for(dilated.q, pass);
    TapBand bands[TAP_BANDS_MAX];
    if (const int nb = tap_bands(p, pass, bands)) {  // partial results of every band (forward, input gradient) + the most a band needs
        const size_t esize = p.dtype == PHX_F32 ? 4 : 2;
        const size_t count = pass == PHX_PASS_FWD ? (size_t)4 * p.n * p.co * p.ho * p.wo : (size_t)4 * p.n * p.ci * p.h * p.w;
        size_t most = 0;
        for (int b = 0; b < nb; ++b) {
            long tap_offset = 0;
            most = std::max(most, workspace_for(band_problem(p, bands[b], tap_offset), pass));
        }
        return (pass == PHX_PASS_BWD_WEIGHTS ? 0 : align_up(nb * count * esize, 256)) + most;
    }
    if (pass == PHX_PASS_BWD_WEIGHTS && wgrad_by_classes(p)) {  // the largest class: its gathered input + its own workspace
        TapClass ch[TAP_CLASSES_MAX], cw[TAP_CLASSES_MAX];
        const int nh = tap_classes(p.kh, p.dh, p.sh, p.pt, p.ho, ch), nw = tap_classes(p.kw, p.dw, p.sw, p.pl, p.wo, cw);
        const size_t esize = p.dtype == PHX_F32 ? 4 : 2;
        size_t most = 0;
        for (int a = 0; a < nh; ++a)
            for (int b = 0; b < nw; ++b) {
                long tap_offset = 0;
                const Problem q = wgrad_class_problem(p, ch[a], cw[b], tap_offset);
                most = std::max(most, align_up((size_t)4 * p.n * p.ci * q.h * q.w * esize, 256) + workspace_for(q, pass));
            }
        return most;
    }
    S2dView v;
    if (pass != PHX_PASS_BWD_DATA && s2d_view(p, v)) return v.x2_bytes + v.w2_bytes + workspace_plain(v.q, pass);
    Problem q;
    size_t xs_bytes = 0;
    if (pass != PHX_PASS_BWD_DATA && subsample_view(p, q, xs_bytes)) {
        const int Z = pass == PHX_PASS_FWD ? corr_slices(q, pass) : 0;  // (the unit-stride problem on the subsampled copy is sliced like any other)
        if (!Z) return xs_bytes + workspace_plain(q, pass);
        const SlicedCorr sc(q, pass, Z);
        return xs_bytes + sc.partial_bytes + (size_t)Z * workspace_plain(sc.q, pass);
    }
    if (const int Z = corr_slices(p, pass)) {
        const SlicedCorr sc(p, pass, Z);
        return sc.partial_bytes + (size_t)Z * workspace_plain(sc.q, pass);
    }
    if (const int Z = pass == PHX_PASS_BWD_DATA ? phase_slices(p) : 0) {
        // phase buffers + the most that a phase takes for its partial tensors and the packed sub-filters of its slices
        const size_t esize = p.dtype == PHX_F32 ? 4 : 2;
        size_t bufs = 0, most = 0;
        for (int a = 0; a < p.sh; ++a)
            for (int b = 0; b < p.sw; ++b) {
                const PhaseAxis ah = phase_axis(a, p.h, p.kh, p.dh, p.sh, p.pt), aw = phase_axis(b, p.w, p.kw, p.dw, p.sw, p.pl);
                if (!ah.taps || !aw.taps || !ah.size || !aw.size) continue;
                bufs += align_up((size_t)4 * p.n * p.ci * ah.size * aw.size * esize, 256);
                const SlicedCorr sc(p, pass, Z, (long)ah.size * aw.size);
                Corr c;
                FwdPlan pl;
                int pw = 0;
                if (!plan_corr(phase_corr(sc.q, ah, aw), p.mode, use_f16_mfma(p, pass), c, pl, pw)) return 0;
                most = std::max(most, sc.partial_bytes + (size_t)Z * align_up(pl.wpk_bytes, 256));
            }
        return bufs + most;
    }
    return workspace_plain(p, pass);
}

static void s2d_rearrange_input(const Problem& p, const S2dView& v, const void* x, void* x2, hipStream_t st) {
    S2dArgs a;
    a.src = x; a.dst = x2; a.planes = (p.real_input ? 1L : 4L) * p.n * p.ci; a.H = p.h; a.W = p.w; a.H2 = v.q.h; a.W2 = v.q.w;
    launch_s2d_input(p.dtype == PHX_F16, a, st);
}

static int do_fwd(const Problem& p, hipStream_t st, const void* x, const void* w, const void* bias, void* y, void* ws, size_t wsb);
static int do_bwd_data(const Problem& p, hipStream_t st, const void* g, const void* w, void* dx, void* ws, size_t wsb);
// Forward (map == MAP_FWD: in = x) or input gradient by tap bands: a pass per band into its partial tensor, then their sum
static int run_banded(const Problem& p, const TapBand* bands, int nb, int map, hipStream_t st, const void* in, const void* w, const void* bias,
                      void* out, void* ws, size_t wsb) {
    const bool dry = g_pack.dry();
    const size_t esize = p.dtype == PHX_F32 ? 4 : 2;
    const long count = map == MAP_FWD ? 4L * p.n * p.co * p.ho * p.wo : 4L * p.n * p.ci * p.h * p.w;
    const size_t partial_bytes = align_up((size_t)nb * count * esize, 256);
    if (!dry && (wsb < partial_bytes || !ws)) return PHX_ERR_WORKSPACE;
    char* partial = static_cast<char*>(ws);
    g_name_prefix = "band_";
    for (int b = 0; b < nb; ++b) {
        long tap_offset = 0;
        const Problem q = band_problem(p, bands[b], tap_offset);
        const void* wb = at_bytes(w, (size_t)tap_offset * esize);
        void* part = dry ? nullptr : partial + (size_t)b * count * esize;
        void* rest = dry ? nullptr : partial + partial_bytes;
        const int rc = map == MAP_FWD ? do_fwd(q, st, in, wb, nullptr, part, rest, dry ? 0 : wsb - partial_bytes)
                                      : do_bwd_data(q, st, in, wb, part, rest, dry ? 0 : wsb - partial_bytes);
        if (rc != PHX_OK) { g_name_prefix = ""; return rc; }
    }
    g_name_prefix = "";
    if (dry) return PHX_OK;
    const bool add = map == MAP_DGRAD && g_addend.dx == out && g_addend.ptr && !g_addend.fused;
    launch_slice_sum(p.dtype == PHX_F16, partial, nb, count, out, bias, add ? g_addend.ptr : nullptr,
                     map == MAP_FWD ? p.ho * p.wo : p.h * p.w, map == MAP_FWD ? p.co : p.ci, count / 4, st);
    PHX_HIP(hipGetLastError());
    if (add) g_addend.fused = true;
    return PHX_OK;
}

// One forward (map == MAP_FWD: in = x) or input-gradient pass in Z reduction slices (see corr_slices)
// (ah, aw: one phase of a strided input gradient, out = that phase's buffer)
static int run_sliced(const Problem& p, int Z, int map, hipStream_t st, const void* in, const void* w, const void* bias, void* out,
                      void* ws, size_t wsb, const PhaseAxis* ah = nullptr, const PhaseAxis* aw = nullptr) {
    const int pass = map == MAP_FWD ? PHX_PASS_FWD : PHX_PASS_BWD_DATA;
    const long plane = ah ? (long)ah->size * aw->size : map == MAP_FWD ? (long)p.ho * p.wo : (long)p.h * p.w;
    const SlicedCorr sc(p, pass, Z, ah ? plane : 0);
    const bool dry = g_pack.dry();
    if (!dry && (wsb < sc.partial_bytes || !ws)) return PHX_ERR_WORKSPACE;
    char* partial = static_cast<char*>(ws);
    g_batch = sc.steps;
    const int rc = run_corr(sc.q, ah ? phase_corr(sc.q, *ah, *aw) : map == MAP_FWD ? corr_forward(sc.q) : corr_dgrad(sc.q), map, st, in, w, nullptr, dry ? nullptr : partial,
                            dry ? nullptr : partial + sc.partial_bytes, dry ? 0 : wsb - sc.partial_bytes);
    g_batch = GroupBatch{};
    if (rc != PHX_OK || dry) return rc;
    const bool add = map == MAP_DGRAD && g_addend.dx == out && g_addend.ptr && !g_addend.fused;
    launch_slice_sum(p.dtype == PHX_F16, partial, Z, sc.count, out, bias, add ? g_addend.ptr : nullptr,
                     (int)plane, map == MAP_FWD ? p.co : p.ci, sc.count / 4, st);
    PHX_HIP(hipGetLastError());
    if (add) g_addend.fused = true;
    const size_t len = strlen(g_name_buf);
    if (g_last_kernel == g_name_buf && len < sizeof(g_name_buf)) snprintf(g_name_buf + len, sizeof(g_name_buf) - len, "_kslices%d", Z);
    return PHX_OK;
}

static int do_fwd(const Problem& p, hipStream_t st, const void* x, const void* w, const void* bias, void* y, void* ws,
                  size_t wsb) {
    if (is_empty(p)) return PHX_OK;  // the reference returns silently on empty input (src/conv2d.hpp:81-82)
    const bool dry = g_pack.dry();
    if (!dry && (!x || !w || !y || (p.has_bias && !bias))) return PHX_ERR_INVALID_ARGUMENT;
    const void* b = p.has_bias ? bias : nullptr;
    PatchView patches;
    if (patch_view(p, PHX_PASS_FWD, patches)) {
        if (!dry && (wsb < patches.x_bytes || !ws)) return PHX_ERR_WORKSPACE;
        if (!dry) {
            patch_depth(p, patches, x, ws, false, st);
            PHX_HIP(hipGetLastError());
        }
        g_name_prefix = "patch_";
        const int rc = do_fwd(patches.q, st, ws, w, b, y, dry ? nullptr : static_cast<char*>(ws) + patches.x_bytes, dry ? 0 : wsb - patches.x_bytes);
        g_name_prefix = "";
        return rc;
    }
    DilationView dilated;
    if (dilation_view(p, PHX_PASS_FWD, dilated)) {
        const size_t tensors = dilated.x_bytes + dilated.y_bytes;
        if (!dry && (wsb < tensors || !ws)) return PHX_ERR_WORKSPACE;
        char* x2 = static_cast<char*>(ws);
        char* y2 = dry ? nullptr : x2 + dilated.x_bytes;
        if (!dry) {
            dilation_phases(p, dilated, true, x, x2, false, st);
            PHX_HIP(hipGetLastError());
        }
        g_name_prefix = "dil_";
        const int rc = do_fwd(dilated.q, st, x2, w, b, y2, dry ? nullptr : y2 + dilated.y_bytes, dry ? 0 : wsb - tensors);
        g_name_prefix = "";
        if (rc != PHX_OK || dry) return rc;
        dilation_phases(p, dilated, false, y2, y, true, st);
        PHX_HIP(hipGetLastError());
        return PHX_OK;
    }
    TapBand bands[TAP_BANDS_MAX];
    if (const int nb = tap_bands(p, PHX_PASS_FWD, bands)) return run_banded(p, bands, nb, MAP_FWD, st, x, w, b, y, ws, wsb);
    S2dView v;
    if (s2d_view(p, v)) {
        // (the rearranged filter of this path is itself made per call: no prepacked form)
        if (g_pack.mode != PackSession::OFF) return PHX_ERR_NOT_SUPPORTED;
        if (wsb < v.x2_bytes + v.w2_bytes || !ws) return PHX_ERR_WORKSPACE;
        char* x2 = static_cast<char*>(ws);
        char* w2 = x2 + v.x2_bytes;
        s2d_rearrange_input(p, v, x, x2, st);
        S2dFilterArgs fa = v.fa;
        fa.w = w; fa.w2 = w2;
        launch_s2d_filter(p.dtype == PHX_F16, fa, false, st);
        PHX_HIP(hipGetLastError());
        g_name_prefix = "s2d_";
        const int rc = run_corr(v.q, corr_forward(v.q), MAP_FWD, st, x2, w2, b, y, w2 + v.w2_bytes,
                                wsb - v.x2_bytes - v.w2_bytes);
        g_name_prefix = "";
        return rc;
    }
    Problem q;
    size_t xs_bytes = 0;
    if (subsample_view(p, q, xs_bytes)) {
        if (!dry) {
            if (wsb < xs_bytes || !ws) return PHX_ERR_WORKSPACE;
            subsample_input(p, x, ws, st);
            PHX_HIP(hipGetLastError());
        }
        g_name_prefix = "sub_";
        void* rest = dry ? nullptr : static_cast<char*>(ws) + xs_bytes;
        const int Z = corr_slices(q, PHX_PASS_FWD);
        const int rc = Z ? run_sliced(q, Z, MAP_FWD, st, ws, w, b, y, rest, dry ? 0 : wsb - xs_bytes)
                         : run_corr(q, corr_forward(q), MAP_FWD, st, ws, w, b, y, rest, dry ? 0 : wsb - xs_bytes);
        g_name_prefix = "";
        return rc;
    }
    if (const int Z = corr_slices(p, PHX_PASS_FWD)) return run_sliced(p, Z, MAP_FWD, st, x, w, b, y, ws, wsb);
    const Corr c = corr_forward(p);
    return run_corr(p, c, MAP_FWD, st, x, w, b, y, ws, wsb);
}

static int do_bwd_data(const Problem& p, hipStream_t st, const void* g, const void* w, void* dx, void* ws, size_t wsb) {
    if (is_empty(p)) return PHX_OK;
    const bool dry = g_pack.dry();
    if (!dry && (!g || !w || !dx)) return PHX_ERR_INVALID_ARGUMENT;
    PatchView patches;
    if (patch_view(p, PHX_PASS_BWD_DATA, patches)) {
        if (!dry && (wsb < patches.x_bytes || !ws)) return PHX_ERR_WORKSPACE;
        g_name_prefix = "patch_";
        const int rc = do_bwd_data(patches.q, st, g, w, ws, dry ? nullptr : static_cast<char*>(ws) + patches.x_bytes, dry ? 0 : wsb - patches.x_bytes);
        g_name_prefix = "";
        if (rc != PHX_OK || dry) return rc;
        patch_depth(p, patches, ws, dx, true, st);
        PHX_HIP(hipGetLastError());
        return PHX_OK;
    }
    DilationView dilated;
    if (dilation_view(p, PHX_PASS_BWD_DATA, dilated)) {
        const size_t tensors = dilated.x_bytes + dilated.y_bytes;
        if (!dry && (wsb < tensors || !ws)) return PHX_ERR_WORKSPACE;
        char* dx2 = static_cast<char*>(ws);
        char* g2 = dry ? nullptr : dx2 + dilated.x_bytes;
        if (!dry) {
            dilation_phases(p, dilated, false, g, g2, false, st);
            PHX_HIP(hipGetLastError());
        }
        g_name_prefix = "dil_";
        const int rc = do_bwd_data(dilated.q, st, g2, w, dx2, dry ? nullptr : g2 + dilated.y_bytes, dry ? 0 : wsb - tensors);
        g_name_prefix = "";
        if (rc != PHX_OK || dry) return rc;
        dilation_phases(p, dilated, true, dx2, dx, true, st);
        PHX_HIP(hipGetLastError());
        return PHX_OK;
    }
    TapBand bands[TAP_BANDS_MAX];
    if (const int nb = tap_bands(p, PHX_PASS_BWD_DATA, bands)) return run_banded(p, bands, nb, MAP_DGRAD, st, g, w, nullptr, dx, ws, wsb);
    if (dgrad_by_phases(p)) {
        const size_t esize = p.dtype == PHX_F32 ? 4 : 2;
        PhaseMergeArgs m;
        m.buf = ws; m.dx = dx; m.planes = 4L * p.n * p.ci; m.H = p.h; m.W = p.w; m.sh = p.sh; m.sw = p.sw;
        size_t bufs = 0;
        for (int i = 0; i < PHASES_MAX; ++i) m.off[i] = -1;
        for (int a = 0; a < p.sh; ++a)
            for (int b = 0; b < p.sw; ++b) {
                const PhaseAxis ah = phase_axis(a, p.h, p.kh, p.dh, p.sh, p.pt), aw = phase_axis(b, p.w, p.kw, p.dw, p.sw, p.pl);
                if (!ah.taps || !aw.taps || !ah.size || !aw.size) continue;
                m.off[a * p.sw + b] = (long)(bufs / esize);
                bufs += align_up((size_t)4 * p.n * p.ci * ah.size * aw.size * esize, 256);
            }
        if (dry) { ws = nullptr; wsb = bufs = 0; }  // (only the packing calls of the phases matter)
        else if (wsb < bufs || !ws) return PHX_ERR_WORKSPACE;
        char* base = static_cast<char*>(ws);
        const int Z = phase_slices(p);
        g_name_prefix = "phase_";
        for (int a = 0; a < p.sh; ++a)
            for (int b = 0; b < p.sw; ++b) {
                if (m.off[a * p.sw + b] < 0) continue;
                const PhaseAxis ah = phase_axis(a, p.h, p.kh, p.dh, p.sh, p.pt), aw = phase_axis(b, p.w, p.kw, p.dw, p.sw, p.pl);
                void* phase_out = dry ? nullptr : base + m.off[a * p.sw + b] * esize;
                const int rc = Z ? run_sliced(p, Z, MAP_DGRAD, st, g, w, nullptr, phase_out, dry ? nullptr : base + bufs, wsb - bufs, &ah, &aw)
                                 : run_corr(p, phase_corr(p, ah, aw), MAP_DGRAD, st, g, w, nullptr, phase_out, dry ? nullptr : base + bufs,
                                            wsb - bufs);
                if (rc != PHX_OK) { g_name_prefix = ""; return rc; }
            }
        g_name_prefix = "";
        if (dry) return PHX_OK;
        launch_phase_merge(p.dtype == PHX_F16, m, st);
        PHX_HIP(hipGetLastError());
        return PHX_OK;
    }
    if (const int Z = corr_slices(p, PHX_PASS_BWD_DATA)) return run_sliced(p, Z, MAP_DGRAD, st, g, w, nullptr, dx, ws, wsb);
    const Corr c = corr_dgrad(p);
    return run_corr(p, c, MAP_DGRAD, st, g, w, nullptr, dx, ws, wsb);
}

static int do_bwd_weights(const Problem& p, hipStream_t st, const void* x, const void* g, void* dw, void* ws,
                          size_t wsb) {
    if (!dw) return PHX_ERR_INVALID_ARGUMENT;
    if (is_empty(p)) {  // the reference zeroes the filter gradient on empty input (src/conv2d.hpp:341-344)
        const size_t bytes = (size_t)4 * p.fs.wcs * (p.dtype == PHX_F32 ? 4 : 2);
        launch_fill_zero(dw, bytes, st);
        PHX_HIP(hipGetLastError());
        return PHX_OK;
    }
    if (!x || !g) return PHX_ERR_INVALID_ARGUMENT;
    PatchView patches;
    if (patch_view(p, PHX_PASS_BWD_WEIGHTS, patches)) {
        if (wsb < patches.x_bytes || !ws) return PHX_ERR_WORKSPACE;
        patch_depth(p, patches, x, ws, false, st);
        PHX_HIP(hipGetLastError());
        g_name_prefix = "patch_";
        const int rc = do_bwd_weights(patches.q, st, ws, g, dw, static_cast<char*>(ws) + patches.x_bytes, wsb - patches.x_bytes);
        g_name_prefix = "";
        return rc;
    }
    DilationView dilated;
    if (dilation_view(p, PHX_PASS_BWD_WEIGHTS, dilated)) {
        const size_t tensors = dilated.x_bytes + dilated.y_bytes;
        if (wsb < tensors || !ws) return PHX_ERR_WORKSPACE;
        char* x2 = static_cast<char*>(ws);
        char* g2 = x2 + dilated.x_bytes;
        dilation_phases(p, dilated, true, x, x2, false, st);
        dilation_phases(p, dilated, false, g, g2, false, st);
        PHX_HIP(hipGetLastError());
        g_name_prefix = "dil_";
        const int rc = do_bwd_weights(dilated.q, st, x2, g2, dw, g2 + dilated.y_bytes, wsb - tensors);
        g_name_prefix = "";
        return rc;
    }
    TapBand bands[TAP_BANDS_MAX];
    if (const int nb = tap_bands(p, PHX_PASS_BWD_WEIGHTS, bands)) {  // a band's filter gradient is its block of dw
        if (wsb < workspace_for(p, PHX_PASS_BWD_WEIGHTS) || (!ws && wsb)) return PHX_ERR_WORKSPACE;  // (refused as a whole)
        const size_t esize = p.dtype == PHX_F32 ? 4 : 2;
        g_name_prefix = "band_";
        for (int b = 0; b < nb; ++b) {
            long tap_offset = 0;
            const Problem q = band_problem(p, bands[b], tap_offset);
            const int rc = do_bwd_weights(q, st, x, g, static_cast<char*>(dw) + (size_t)tap_offset * esize, ws, wsb);
            if (rc != PHX_OK) { g_name_prefix = ""; return rc; }
        }
        g_name_prefix = "";
        return PHX_OK;
    }
    if (wgrad_by_classes(p)) {
        TapClass ch[TAP_CLASSES_MAX], cw[TAP_CLASSES_MAX];
        const int nh = tap_classes(p.kh, p.dh, p.sh, p.pt, p.ho, ch), nw = tap_classes(p.kw, p.dw, p.sw, p.pl, p.wo, cw);
        const size_t esize = p.dtype == PHX_F32 ? 4 : 2;
        // (refused as a whole: a class that ran would have written its taps of dw)
        if (wsb < workspace_for(p, PHX_PASS_BWD_WEIGHTS) || !ws) return PHX_ERR_WORKSPACE;
        for (int a = 0; a < nh; ++a)
            for (int b = 0; b < nw; ++b) {
                long tap_offset = 0;
                const Problem q = wgrad_class_problem(p, ch[a], cw[b], tap_offset);
                const size_t xg_bytes = align_up((size_t)4 * p.n * p.ci * q.h * q.w * esize, 256);
                StridedGatherArgs ga;
                ga.src = x; ga.dst = ws; ga.planes = 4L * p.n * p.ci; ga.H = p.h; ga.W = p.w; ga.H2 = q.h; ga.W2 = q.w;
                ga.sh = p.sh; ga.sw = p.sw; ga.oh = ch[a].origin; ga.ow = cw[b].origin;
                launch_strided_gather(p.dtype == PHX_F16, ga, st);
                PHX_HIP(hipGetLastError());
                g_name_prefix = "class_";
                const int rc = do_bwd_weights(q, st, ws, g, static_cast<char*>(dw) + tap_offset * (long)esize, static_cast<char*>(ws) + xg_bytes,
                                              wsb - xg_bytes);
                g_name_prefix = "";
                if (rc != PHX_OK) return rc;
            }
        return PHX_OK;
    }
    S2dView v;
    if (s2d_view(p, v)) {
        if (wsb < v.x2_bytes + v.w2_bytes || !ws) return PHX_ERR_WORKSPACE;
        char* x2 = static_cast<char*>(ws);
        char* dw2 = x2 + v.x2_bytes;
        s2d_rearrange_input(p, v, x, x2, st);
        g_name_prefix = "s2d_";
        const int rc = run_wgrad(v.q, st, x2, g, dw2, dw2 + v.w2_bytes, wsb - v.x2_bytes - v.w2_bytes);
        g_name_prefix = "";
        if (rc != PHX_OK) return rc;
        S2dFilterArgs fa = v.fa;
        fa.w = dw; fa.w2 = dw2;
        launch_s2d_filter(p.dtype == PHX_F16, fa, true, st);
        PHX_HIP(hipGetLastError());
        return PHX_OK;
    }
    Problem q;
    size_t xs_bytes = 0;
    if (subsample_view(p, q, xs_bytes)) {
        if (wsb < xs_bytes || !ws) return PHX_ERR_WORKSPACE;
        subsample_input(p, x, ws, st);
        PHX_HIP(hipGetLastError());
        g_name_prefix = "sub_";
        const int rc = run_wgrad(flatten_pointwise(q), st, ws, g, dw, static_cast<char*>(ws) + xs_bytes, wsb - xs_bytes);
        g_name_prefix = "";
        return rc;
    }
    const Problem f = flatten_pointwise(p);
    return run_wgrad(f, st, x, g, dw, ws, wsb);
}

}  // namespace phx

using namespace phx;

extern "C" {

const char* phx_status_string(int status) {
    switch (status) {
        case PHX_OK: return "ok";
        case PHX_ERR_INVALID_ARGUMENT: return "invalid argument";
        case PHX_ERR_NOT_SUPPORTED: return "not supported";
        case PHX_ERR_WORKSPACE: return "workspace too small";
        case PHX_ERR_RUNTIME: return "HIP runtime error";
        case PHX_ERR_SCRATCH_LIMIT: return "request exceeds the built-in scratch buffer of the no-allocation entry point";
    }
    return "unknown status";
}

const char* phx_last_kernel_name(void) { return g_last_kernel; }

int phx_init(void) { return device_state(nullptr); }

int phx_plan_cache_stats(long* entries, long* evictions) {
    std::lock_guard<std::mutex> lock(g_plan_mutex);
    if (entries) *entries = g_plan_memo_sizes[0] + g_plan_memo_sizes[1];
    if (evictions) *evictions = g_plan_evictions.load();
    return PHX_OK;
}

int phx_tuning_reload(void) {
    std::lock_guard<std::mutex> lock(g_plan_mutex);
    (void)tune();  // (so that a first read cannot race with this one)
    g_tune.read();
    ++g_plan_generation;
    return PHX_OK;
}

int phx_profile_enable(int capacity) {
    std::lock_guard<std::mutex> lock(g_prof_mutex);
    g_prof.on = false;
    g_prof.used = 0;
    if (capacity <= 0) return PHX_OK;
    while ((int)g_prof.ev.size() < 2 * capacity) {
        hipEvent_t e;
        PHX_HIP(hipEventCreate(&e));
        g_prof.ev.push_back(e);
    }
    g_prof.on = true;
    return PHX_OK;
}

int phx_profile_collect(float* milliseconds, int max_count, int* count) {
    if (!count || (max_count > 0 && !milliseconds)) return PHX_ERR_INVALID_ARGUMENT;
    std::lock_guard<std::mutex> lock(g_prof_mutex);
    const int n = std::min(g_prof.used, max_count);
    for (int i = 0; i < n; ++i) {
        PHX_HIP(hipEventSynchronize(g_prof.ev[2 * i + 1]));
        PHX_HIP(hipEventElapsedTime(&milliseconds[i], g_prof.ev[2 * i], g_prof.ev[2 * i + 1]));
    }
    *count = n;
    g_prof.used = 0;
    return PHX_OK;
}

// Grouped convolution (groups passed on to the scalar convolutions in the reference,
// src/backend/onednn/conv2d.hpp:116-137): the groups are independent convolutions on channel slices of the
// same tensors; each runs as a problem of its own whose tensors are views (byte offsets below) with the whole
// tensors' image strides.  An empty problem runs once: it only zeroes the filter gradient, all of it.
struct GroupOffsets {
    size_t x, y, w, b;  // bytes from one group's slice to the next: input, output, filter, bias
    int runs;
    explicit GroupOffsets(const Problem& p) {
        const size_t esize = p.dtype == PHX_F32 ? 4 : 2;
        x = (size_t)p.ci * p.h * p.w * esize;
        y = (size_t)p.co * p.ho * p.wo * esize;
        w = (size_t)p.co * p.fs.so * esize;
        b = (size_t)p.co * esize;
        runs = is_empty(p) ? 1 : p.groups;
    }
    static const void* at(const void* ptr, size_t off) { return ptr ? static_cast<const char*>(ptr) + off : nullptr; }
    static void* at(void* ptr, size_t off) { return ptr ? static_cast<char*>(ptr) + off : nullptr; }
};

struct GroupBatchScope {  // all groups in one launch per kernel (see group_batchable); lasts for one run of a pass
    explicit GroupBatchScope(const Problem& p) {
        const GroupOffsets o(p);
        g_batch.n = o.runs; g_batch.x = o.x; g_batch.y = o.y; g_batch.w = o.w; g_batch.b = o.b;
    }
    ~GroupBatchScope() { g_batch = GroupBatch{}; }
};

// Channels-last activations (DataFormat::NHWC, src/backend/tensor.hpp:17-31): the kernels read and write
// channels-first planes, so such a call keeps channels-first copies of its input-side and output-side activation
// tensors at the front of the workspace and transposes on the way in and out.
struct ChannelsLast {
    size_t x_bytes = 0, y_bytes = 0;
    long x_rows = 0, y_rows = 0;
    explicit ChannelsLast(const Problem& p) {
        if (!p.nhwc) return;
        const size_t esize = p.dtype == PHX_F32 ? 4 : 2;
        x_rows = (p.real_input ? 1L : 4L) * p.n;
        y_rows = 4L * p.n;
        x_bytes = ((size_t)x_rows * p.ci_mem * p.h * p.w * esize + 255) / 256 * 256;
        y_bytes = ((size_t)y_rows * p.co_mem * p.ho * p.wo * esize + 255) / 256 * 256;
    }
    size_t bytes() const { return x_bytes + y_bytes; }
    // caller's input-side tensor -> planes, and back
    void x_in(const Problem& p, const void* x, void* planes, hipStream_t st) const {
        launch_transpose(p.dtype == PHX_F16, TransposeArgs{x, planes, x_rows, p.h * p.w, p.ci_mem}, st);
    }
    void x_out(const Problem& p, const void* planes, void* x, hipStream_t st) const {
        launch_transpose(p.dtype == PHX_F16, TransposeArgs{planes, x, x_rows, p.ci_mem, p.h * p.w}, st);
    }
    void y_in(const Problem& p, const void* y, void* planes, hipStream_t st) const {
        launch_transpose(p.dtype == PHX_F16, TransposeArgs{y, planes, y_rows, p.ho * p.wo, p.co_mem}, st);
    }
    void y_out(const Problem& p, const void* planes, void* y, hipStream_t st) const {
        launch_transpose(p.dtype == PHX_F16, TransposeArgs{planes, y, y_rows, p.co_mem, p.ho * p.wo}, st);
    }
};

// Channels-last windowed convolutions (3x3 and other multi-tap filters; any stride forward, unit stride backward) whose
// forward / input-gradient plan is the chunk-staging fp16 kernel run on the caller's tensors as they are: that kernel's LDS layout is
// [position][8 channels], which IS the channels-last order, so its staging copies 16-byte entries without the
// channel transpose the channels-first form needs, and the epilogue stores 16 consecutive channels of a pixel per
// lane.  Everything else channels-last (the filter gradient, strides, groups, fp32) keeps the transposes.
// A chunk of 16 channels is only 32 contiguous bytes per position, so the staging loads of this form touch many more
// cache lines per instruction than the channels-first ones; the kernel is 0-5 % faster than the channels-first one
// at 64 and 128 channels and 5-12 % slower at 256 and 512 (3x3; 56x56 .. 7x7 images), while the two transposes it
// saves cost in proportion to the tensors, not to the arithmetic.  Calls whose arithmetic per tensor byte
// (channels x taps) is beyond what was measured to pay (256 channels, 3x3) keep the transposes;
// PHX_TUNE_WINCL_MAX moves that bound, PHX_TUNE_NOWINCL switches the direct form off.
namespace phx {
static bool nhwc_window_native(const Problem& p, int pass) {
    if (!p.nhwc || (pass != PHX_PASS_FWD && pass != PHX_PASS_BWD_DATA) || is_empty(p) || is_pointwise_unit(p)) return false;
    if (p.real_input || p.groups != 1 || tune().nowincl || !use_f16_mfma(p, pass)) return false;
    // (a strided forward pass reads its staged window with the stride, whatever the memory order; a strided input
    // gradient runs by phases or on zero-inserted windows, neither of which is staged in chunks)
    if ((p.sh != 1 || p.sw != 1) && pass != PHX_PASS_FWD) return false;
    if ((long)std::max(p.ci, p.co) * p.kh * p.kw > tune().wincl_max) return false;
    if (p.ci % 8 != 0 || p.co % 8 != 0 || p.ci_mem != p.ci || p.co_mem != p.co) return false;  // whole 16-byte entries, 8-byte stores
    S2dView v;
    if (pass == PHX_PASS_FWD && s2d_view(p, v)) return false;
    if (pass == PHX_PASS_BWD_DATA && dgrad_by_phases(p)) return false;
    Corr c;
    FwdPlan pl;
    int pw = 0;
    if (!plan_corr(pass == PHX_PASS_FWD ? corr_forward(p) : corr_dgrad(p), p.mode, true, c, pl, pw)) return false;
    if (!(pl.lds_filters && pl.chunks && !pl.pwx && pw == 0)) return false;
    // a small batch on a deep layer gains more from reduction slices (corr_slices), which run on channels-first copies:
    // the copies of so small a problem cost next to nothing; so do dilated windows from their dilation phases
    Problem planes = p;
    planes.nhwc = false;
    DilationView dilated;
    PatchView patches;
    TapBand bands[TAP_BANDS_MAX];
    return corr_slices(planes, pass) == 0 && !dilation_view(planes, pass, dilated) && !patch_view(planes, pass, patches) && !tap_bands(planes, pass, bands);
}
}  // namespace phx

// The filter gradient of a channels-last call runs on the caller's tensors where its plan is the fp16 kernel with
// 64x64 channel tiles, unit stride and one or three taps per workgroup (more than 32 channels on either side): that
// kernel's channels-last staging transposes 8x8 blocks in registers on the way to LDS (qconv_wgrad_f16_kernel, CL).
static bool nhwc_wgrad_native(const Problem& p) {
    if (!p.nhwc || is_empty(p) || p.real_input || p.groups != 1 || p.sh != 1 || p.sw != 1 || tune().nowincl) return false;
    if (window_beyond_staging(p)) return false;  // (the vector-ALU kernels, or the dilation phases of channels-first copies)
    if (p.ci % 8 != 0 || p.co % 8 != 0 || p.ci_mem != p.ci || p.co_mem != p.co) return false;
    const Problem f = flatten_pointwise(p);
    if (!wgrad_on_f16_mfma(f)) return false;
    WgPlan pl;
    if (!plan_wgrad(f, true, pl)) return false;
    return !pl.realx && pl.kmode == 16 && pl.MT == 2 && pl.NT == 2 && pl.SW == 1 && (pl.TPW == 1 || pl.TPW == 3);
}

// Grouped convolutions whose groups hold very few channels (depthwise convolutions first of all) run on the vector-ALU
// kernels of phx_launch_thin.hip, all groups by one launch per pass, straight on the caller's channels-first tensors
// and filter.  A matrix-core tile spans 32 x 32 channels of one group and costs the same whatever it holds; the
// vector-ALU threads cost in proportion to the channel pairs of a group (input x output channels).  Measured against
// the matrix-core path with merged groups (merged_groups below; 128 channels, 28x28, N=32, fwd / dgrad / wgrad us):
// depthwise 3x3 29 / 28 / 54 against 49 / 50 / 54, 5x5 (96 channels, 56x56) 128 / 122 / 231 against 261 / 263 / 610,
// 2 x 2 channels per group 45 / 42 / 73 against 48 / 47 / 53, 4 x 4 71 / 67 / 111 against 46 / 45 / 51: up to four
// pairs per group run here.  PHX_TUNE_THIN_MAX moves the bound.
//
// The same kernels are the way out for filters whose window does not fit the matrix-core kernels' staging: those
// stage one window position per thread, so the window of a single output position -- ((kh-1) dh + 1) rows of
// ((kw-1) dw + 1) columns, rounded up to whole 8-position chunks -- must not exceed 256 positions (a 7x7 filter at
// dilation 3, a 17x17 one).  Such convolutions, grouped or not, run here at vector-ALU speed rather than not at all.
// (window_beyond_staging; dilated ones that dilation_view can rewrite run as undilated convolutions instead)
static bool thin_groups(const Problem& p, int pass) {
    if (is_empty(p) || p.ho <= 0 || p.wo <= 0) return false;
    if ((long)p.kh * p.kw > 2048 || std::max(p.ci_mem, p.co_mem) > 65535) return false;  // (a filter chunk in LDS; grid rows)
    if (tune().direct) return true;
    DilationView dilated;
    PatchView patches;
    TapBand bands[TAP_BANDS_MAX];
    const long pairs = (long)p.ci * p.co;
    // (the rule for filter gradients of few channels in fp32 arithmetic, see below)
    const bool few_fp32 = pass == PHX_PASS_BWD_WEIGHTS && p.groups <= 1 && tune().thin_max32 > 0 && !wgrad_on_f16_mfma(flatten_pointwise(p)) &&
                          pairs <= (p.kh * p.kw > 1 ? 512 : 128);
    if (window_beyond_staging(p))
        return few_fp32 || (!dilation_view(p, pass, dilated) && !patch_view(p, pass, patches) && !tap_bands(p, pass, bands));
    // at their staging limit the matrix-core kernels work on tiles of a single output position (a grouped 16x16 filter,
    // 8 groups of 32 channels: 1.1 s for an input gradient): what the tap bands do not take runs here as well
    if (window_positions(p) > 224 && (p.groups > 1 || p.real_input))
        return !dilation_view(p, pass, dilated) && !patch_view(p, pass, patches);
    // The filter gradient in fp32 arithmetic works on 64 x 64 channel tiles whatever the layer holds: its time follows
    // the pixels and taps alone (3x3, 56x56, N=64: 1.39 ms from 8 to 64 channels), that of the vector-ALU kernel the
    // channel pairs too -- 8 -> 8 channels 0.11 ms, 16 -> 16 0.35, 3 -> 64 0.29, 24 -> 24 0.77, 32 -> 32 1.20; a
    // single tap: 16 -> 16 0.18 against 0.17.  Layers of few channels, grouped or not, run it here.
    if (pass == PHX_PASS_BWD_WEIGHTS && p.groups <= 1 && tune().thin_max32 > 0 && !wgrad_on_f16_mfma(flatten_pointwise(p)))
        return few_fp32;
    if (p.groups <= 1) return false;
    // Passes in fp32 arithmetic (fp32 tensors, fp16 tensors where the policy says so) have a sixteenth of the fp16
    // matrix-core rate to lose against, and their filter gradient works on 64 x 64 channel tiles: measured like above,
    // 8 x 8 channels per group 159 / 149 / 206 us here against 194 / 193 / 742 merged, 16 x 16 260 / 254 / 346 against
    // 192 / 193 / 745 -- up to 64 pairs per group run here, the filter gradient up to 256.
    if (use_f16_mfma(p, pass)) return pairs <= tune().thin_max;
    return pairs <= (long)tune().thin_max32 * (pass == PHX_PASS_BWD_WEIGHTS ? 4 : 1);
}

static ThinArgs thin_args(const Problem& p) {
    ThinArgs t{};
    t.wcs = p.fs.wcs; t.so = p.fs.so; t.si = p.fs.si; t.skh = p.fs.skh; t.skw = p.fs.skw;
    t.N = p.n; t.groups = p.groups; t.cig = p.ci; t.cog = p.co;
    t.H = p.h; t.W = p.w; t.Ho = p.ho; t.Wo = p.wo;
    t.Kh = p.kh; t.Kw = p.kw; t.sh = p.sh; t.sw = p.sw; t.dh = p.dh; t.dw = p.dw; t.pt = p.pt; t.pl = p.pl;
    t.Z = 1;
    t.real_x = p.real_input ? 1 : 0;
    t.mh = p.sh > 1 ? (unsigned int)(((1ULL << 32) + p.sh - 1) / p.sh) : 0u;
    t.mw = p.sw > 1 ? (unsigned int)(((1ULL << 32) + p.sw - 1) / p.sw) : 0u;
    return t;
}
// the filter gradient's partial sums: [slices][output channel x input channel of its group][tap][4]
static size_t thin_workspace(const Problem& p, int pass) {
    if (pass != PHX_PASS_BWD_WEIGHTS) return 0;
    return align_up((size_t)thin_wgrad_slices(p.dtype == PHX_F16, thin_args(p)) * p.co_mem * p.ci * p.kh * p.kw * 4 * sizeof(float), 256);
}

// (a, b) = (x, w) forward, (grad, w) input gradient, (x, grad) filter gradient; channels-first tensors of all groups
static int run_thin(const Problem& p, int pass, hipStream_t st, const void* a, const void* b, const void* bias, void* out, void* ws,
                    size_t wsb) {
    if (!a || !b || !out || (pass == PHX_PASS_FWD && p.has_bias && !bias)) return PHX_ERR_INVALID_ARGUMENT;
    ThinArgs t = thin_args(p);
    t.in = a; t.out = out;
    if (pass == PHX_PASS_BWD_WEIGHTS) {
        t.grad = b;
        t.Z = thin_wgrad_slices(p.dtype == PHX_F16, t);
        if (thin_workspace(p, pass) > wsb || !ws) return PHX_ERR_WORKSPACE;
        t.partial = static_cast<float*>(ws);
    } else {
        t.w = b;
        t.bias = (pass == PHX_PASS_FWD && p.has_bias) ? bias : nullptr;
    }
    int rc;
    {
        KernelTimer timer(st);
        rc = launch_thin(p.dtype == PHX_F16, pass, t, st);
    }
    if (rc < 0) return PHX_ERR_NOT_SUPPORTED;
    PHX_HIP(hipGetLastError());
    if (pass == PHX_PASS_BWD_WEIGHTS)
        snprintf(g_name_buf, sizeof(g_name_buf), "qconv_wgrad_fma_thin_%s_g%dx%dx%d_k%dx%d%s_z%d", p.dtype == PHX_F32 ? "f32" : "f16", p.groups,
                 p.ci, p.co, p.kh, p.kw, rc == 1 ? "_tile" : "", t.Z);
    else
        snprintf(g_name_buf, sizeof(g_name_buf), "qconv_%s_fma_thin_%s_g%dx%dx%d_k%dx%d%s", pass == PHX_PASS_FWD ? "fwd" : "dgrad",
                 p.dtype == PHX_F32 ? "f32" : "f16", p.groups, p.ci, p.co, p.kh, p.kw, rc == 1 ? "_tile" : rc == 2 ? "_phasetile" : "");
    g_last_kernel = g_name_buf;
    say(p, pass == PHX_PASS_FWD ? "forward (thin groups)" : pass == PHX_PASS_BWD_DATA ? "input gradient (thin groups)" : "filter gradient (thin groups)");
    return PHX_OK;
}

namespace phx {
// A grouped convolution runs ALL its groups in one launch per kernel -- grid rows = groups, every kernel shifting its
// tensors by its row's byte steps (group_view) -- the way the reference hands `groups` to one primitive
// (src/backend/onednn/conv2d.hpp:116-137), wherever the pass is a plain run of the kernels on channel-slice views:
// channels-first tensors, all components present, none of the rewritten forms (space-to-depth, subsampled strided
// pointwise, input gradient by phases), whose rearrangement kernels work on one group's tensors.  Everything else
// runs group after group.  The plans are those of one group, so the results are the same either way.
static bool group_batchable(const Problem& p, int pass) {
    if (p.groups <= 1 || is_empty(p) || p.nhwc || p.real_input || tune().nogroupbatch) return false;
    S2dView v;
    Problem q;
    size_t xs_bytes = 0;
    if (pass != PHX_PASS_BWD_DATA && (s2d_view(p, v) || subsample_view(p, q, xs_bytes))) return false;
    if (pass == PHX_PASS_BWD_DATA && dgrad_by_phases(p)) return false;
    return true;
}
}  // namespace phx

// One pass of a grouped convolution on channels-first tensors of all groups: by one launch per kernel where the pass
// is a plain run of the kernels (group_batchable), group after group otherwise.  (a, b) = (x, w) forward,
// (grad, w) input gradient, (x, grad) filter gradient.
static int groups_pass(const Problem& p, int pass, hipStream_t st, const void* a, const void* b, const void* bias, void* out, void* ws,
                       size_t wsb) {
    const auto one = [&](const void* a_, const void* b_, const void* bias_, void* out_) {
        return pass == PHX_PASS_FWD ? do_fwd(p, st, a_, b_, bias_, out_, ws, wsb)
               : pass == PHX_PASS_BWD_DATA ? do_bwd_data(p, st, a_, b_, out_, ws, wsb) : do_bwd_weights(p, st, a_, b_, out_, ws, wsb);
    };
    if (group_batchable(p, pass)) {
        const GroupBatchScope batch(p);
        return one(a, b, bias, out);
    }
    const GroupOffsets o(p);
    // bytes from a group to the next in the three tensors of the pass
    const size_t sa = pass == PHX_PASS_BWD_DATA ? o.y : o.x, sb = pass == PHX_PASS_BWD_WEIGHTS ? o.y : o.w;
    const size_t so = pass == PHX_PASS_FWD ? o.y : pass == PHX_PASS_BWD_DATA ? o.x : o.w;
    for (int g = 0; g < o.runs; ++g) {
        const int rc = one(o.at(a, g * sa), o.at(b, g * sb), bias ? o.at(bias, g * o.b) : nullptr, o.at(out, g * so));
        if (rc != PHX_OK) return rc;
    }
    return PHX_OK;
}
static size_t groups_workspace(const Problem& p, int pass) {
    return (group_batchable(p, pass) ? (size_t)p.groups : (size_t)1) * workspace_for(p, pass);
}

// Merged groups: a matrix-core tile spans 32 x 32 channels of one group, so groups of fewer channels leave most of
// it empty and still cost a tile each.  m consecutive groups (m the largest divisor of the group count with
// m x channels <= 32) are run as ONE group of m * ci -> m * co channels whose filter is block-diagonal: the
// activation tensors are the same memory, the filter is expanded with zeros (merge_filter_kernel: a few KB; per call, or once with the packed images),
// the filter gradient's diagonal blocks are copied out.  The tile then does m times the arithmetic it needs to, which
// the matrix cores have to spare: 32 groups of 4 x 4 channels (3x3, 28x28, N=32) take the time of 4 groups of 32 x 32.
// Returns m (0: no merging).  Where the group count has no divisor that fills the tile as well, the first
// groups - groups % m groups are merged m at a time and the remaining groups % m as one more (run_merged).
static int merged_groups(const Problem& p, int pass) {
    if (p.groups <= 1 || is_empty(p) || p.real_input || tune().nomerge) return 0;
    // (the filter gradient in fp32 arithmetic works on 64 x 64 channel tiles)
    const int tile = (pass == PHX_PASS_BWD_WEIGHTS && !wgrad_on_f16_mfma(flatten_pointwise(p))) ? 64 : 32;
    const int most = std::min(p.groups, tile / std::max(p.ci, p.co));  // groups that fit a tile
    if (most < 2) return 0;
    int divisor = 1;
    for (int d = 2; d <= most; ++d)
        if (p.groups % d == 0) divisor = d;
    return (divisor > 1 && p.groups / divisor == cdiv(p.groups, most)) ? divisor : most;
}
struct MergedGroups {
    Problem q;            // the merged problem: groups / m groups of m * ci -> m * co channels, channels-first
    size_t filter_bytes;  // the block-diagonal filter (or its gradient), OIHW, at the front of the workspace
    MergeFilterArgs fa;
    MergedGroups(const Problem& p, int m) {
        q = p;
        q.groups = p.groups / m; q.ci = p.ci * m; q.co = p.co * m; q.nhwc = false;
        const long taps = (long)p.kh * p.kw;
        q.fs.skw = 1; q.fs.skh = p.kw; q.fs.si = taps; q.fs.so = (long)q.ci * taps; q.fs.wcs = (long)p.groups * p.co * q.fs.so;
        filter_bytes = align_up((size_t)4 * q.fs.wcs * (p.dtype == PHX_F32 ? 4 : 2), 256);
        fa = MergeFilterArgs{nullptr, nullptr, p.fs.wcs, p.fs.so, p.fs.si, p.fs.skh, p.fs.skw, p.groups * p.co, p.ci, p.co, m, p.kh, p.kw};
    }
    size_t workspace(int pass) const { return filter_bytes + groups_workspace(q, pass); }
};
// (a, b) as in groups_pass, on channels-first tensors.  In a packing session (PackSession) the block-diagonal filter is
// an image like the packed ones: SIZE counts it, RECORD makes it (on the session's stream, ahead of the combined
// packing launch that reads it), USE finds it where RECORD put it.
static int run_merged_part(const Problem& p, int m, int pass, hipStream_t st, const void* a, const void* b, const void* bias, void* out,
                           void* ws, size_t wsb) {
    const MergedGroups mg(p, m);
    const PackSession::Mode session = g_pack.mode;
    void* merged_filter = ws;
    char* inner = static_cast<char*>(ws);
    size_t inner_bytes = wsb;
    if (session == PackSession::OFF || pass == PHX_PASS_BWD_WEIGHTS) {
        if (!ws || wsb < mg.filter_bytes) return PHX_ERR_WORKSPACE;
        inner += mg.filter_bytes;
        inner_bytes -= mg.filter_bytes;
    } else {
        const PackSlot slot = pack_slot(nullptr, 0, mg.filter_bytes);
        if (slot.rc != PHX_OK) return slot.rc;
        merged_filter = slot.dst;  // (null while SIZE only counts)
    }
    MergeFilterArgs fa = mg.fa;
    fa.w2 = merged_filter;
    g_name_suffix_merged = m;
    int rc;
    if (pass == PHX_PASS_BWD_WEIGHTS) {
        rc = groups_pass(mg.q, pass, st, a, b, nullptr, merged_filter, inner, inner_bytes);  // the merged filter gradient, then its diagonal blocks
        if (rc == PHX_OK) {
            fa.w = out;
            launch_merge_filter(p.dtype == PHX_F16, fa, true, st);
        }
    } else {
        fa.w = b;
        if (session == PackSession::OFF) launch_merge_filter(p.dtype == PHX_F16, fa, false, st);
        else if (session == PackSession::RECORD) launch_merge_filter(p.dtype == PHX_F16, fa, false, g_pack.st);
        rc = groups_pass(mg.q, pass, st, a, merged_filter, bias, out, inner, inner_bytes);
    }
    g_name_suffix_merged = 0;
    if (rc != PHX_OK) return rc;
    if (session != PackSession::SIZE) PHX_HIP(hipGetLastError());
    return PHX_OK;
}

// The parts of a merged run: `first` groups merged m at a time, then the `rest` (fewer than m) as one group more.
struct MergedParts {
    Problem head, tail;
    int first, rest;
    MergedParts(const Problem& p, int m) : head(p), tail(p), first(p.groups - p.groups % m), rest(p.groups % m) {
        head.groups = first;
        tail.groups = rest;
    }
};
static size_t merged_workspace(const Problem& p, int m, int pass) {
    const MergedParts parts(p, m);
    size_t bytes = MergedGroups(parts.head, m).workspace(pass);
    if (parts.rest > 1) bytes = std::max(bytes, MergedGroups(parts.tail, parts.rest).workspace(pass));
    if (parts.rest == 1) bytes = std::max(bytes, groups_workspace(parts.tail, pass));
    return bytes;
}
static int run_merged(const Problem& p, int m, int pass, hipStream_t st, const void* a, const void* b, const void* bias, void* out,
                      void* ws, size_t wsb) {
    const MergedParts parts(p, m);
    if (const int rc = run_merged_part(parts.head, m, pass, st, a, b, bias, out, ws, wsb)) return rc;
    if (parts.rest == 0) return PHX_OK;
    // the remaining groups' slices of the three tensors (and of the bias)
    const GroupOffsets o(p);
    const size_t sa = pass == PHX_PASS_BWD_DATA ? o.y : o.x, sb = pass == PHX_PASS_BWD_WEIGHTS ? o.y : o.w;
    const size_t so = pass == PHX_PASS_FWD ? o.y : pass == PHX_PASS_BWD_DATA ? o.x : o.w;
    const void* a2 = o.at(a, parts.first * sa);
    const void* b2 = o.at(b, parts.first * sb);
    const void* bias2 = bias ? o.at(bias, parts.first * o.b) : nullptr;
    void* out2 = o.at(out, parts.first * so);
    if (parts.rest == 1) return groups_pass(parts.tail, pass, st, a2, b2, bias2, out2, ws, wsb);
    return run_merged_part(parts.tail, parts.rest, pass, st, a2, b2, bias2, out2, ws, wsb);
}

// Entry points check their descriptor before they touch the device: an invalid descriptor is an invalid argument
// whether or not a device is present.
static int conv_desc_status(const phx_qconv_desc* desc) {
    if (!desc) return PHX_ERR_INVALID_ARGUMENT;
    phx_qconv_desc q = *desc;
    q.algebra = PHX_QUATERNION;  // (the geometry rules are the same for every algebra)
    Problem p;
    return problem_from_conv(&q, p);
}
static int dense_desc_status(const phx_qdense_desc* desc) {
    if (!desc) return PHX_ERR_INVALID_ARGUMENT;
    phx_qdense_desc q = *desc;
    q.algebra = PHX_QUATERNION;
    Problem p;
    return problem_from_dense(&q, p);
}

int phx_qconv2d_output_hw(const phx_qconv_desc* desc, int32_t* ho, int32_t* wo) {
    Problem p;
    const int rc = problem_from_conv(desc, p);
    if (rc != PHX_OK) return rc;
    if (ho) *ho = p.ho;
    if (wo) *wo = p.wo;
    return PHX_OK;
}

size_t phx_qconv2d_workspace_bytes(const phx_qconv_desc* desc, int pass) {
    if (desc && desc->algebra != PHX_QUATERNION) return algebra_conv_workspace_bytes(desc, pass);
    Problem p;
    if (problem_from_conv(desc, p) != PHX_OK) return 0;
    if (thin_groups(p, pass)) return ChannelsLast(p).bytes() + thin_workspace(p, pass);
    if (nhwc_native(p, pass)) return nhwc_native_workspace(p, pass);
    if (nhwc_window_native(p, pass)) return workspace_for(p, pass);
    if (pass == PHX_PASS_BWD_WEIGHTS && nhwc_wgrad_native(p)) return workspace_for(p, pass);
    if (const int m = merged_groups(p, pass)) return ChannelsLast(p).bytes() + merged_workspace(p, m, pass);
    // (packed images / partial sums of all groups side by side where one launch runs them)
    if (group_batchable(p, pass)) return (size_t)p.groups * workspace_for(p, pass);
    return ChannelsLast(p).bytes() + workspace_for(p, pass);
}

// Small Dense problems (a classifier head, the reference's 128 -> 128 benchmark layer at batch 32) run on plain fp32
// FMA threads: no packing, no workspace, one launch per pass (phx_launch_dense_small.hip).  Up to 16 M quaternion
// products per pass; beyond that the matrix cores win.
static bool dense_is_small(const Problem& p) {
    return !tune().nosmalldense && (double)p.n * p.ci * p.co <= 16.0 * 1024 * 1024 && (long)p.n * std::max(p.ci, p.co) < (1L << 30) &&
           (long)p.ci * p.co < (1L << 30);
}

static int run_dense_small(const Problem& p, int pass, hipStream_t st, const void* a, const void* b, const void* bias, void* out) {
    if (!out || (p.n > 0 && (!a || !b)) || (pass == PHX_PASS_FWD && p.has_bias && !bias)) return PHX_ERR_INVALID_ARGUMENT;
    DenseSmallArgs d{a, b, (pass == PHX_PASS_FWD && p.has_bias) ? bias : nullptr, out, p.fs.wcs, p.fs.so, p.fs.si, p.n, p.ci, p.co};
    int rc;
    {
        KernelTimer timer(st);
        rc = launch_dense_small(p.dtype == PHX_F16, pass, d, st);
    }
    if (rc != 0) return PHX_ERR_NOT_SUPPORTED;
    PHX_HIP(hipGetLastError());
    snprintf(g_name_buf, sizeof(g_name_buf), "qdense_%s_fma_%s_n%d_i%d_o%d",
             pass == PHX_PASS_FWD ? "fwd" : pass == PHX_PASS_BWD_DATA ? "dgrad" : "wgrad", p.dtype == PHX_F32 ? "f32" : "f16", p.n, p.ci, p.co);
    g_last_kernel = g_name_buf;
    say(p, pass == PHX_PASS_FWD ? "forward (dense)" : pass == PHX_PASS_BWD_DATA ? "input gradient (dense)" : "filter gradient (dense)");
    return PHX_OK;
}

// A Dense layer's tensors [4n, units] are those of a channels-last pointwise convolution on ONE image of n x 1
// positions, so the larger fp16 problems run on the channels-last pointwise kernels (streaming operand copies, no
// staged windows) instead of a 1 x 1 convolution on n images of one position each.  PHX_TUNE_NODENSECL keeps the latter.
static bool dense_as_channels_last(const Problem& p, int pass, Problem& q) {
    if (tune().nodensecl || is_empty(p)) return false;
    q = p;
    q.n = 1; q.h = p.n; q.w = 1; q.ho = p.n; q.wo = 1; q.nhwc = true;
    return pass == PHX_PASS_BWD_WEIGHTS ? nhwc_wgrad_native(q) : nhwc_native(q, pass);
}

// The FMA kernels' filter gradient is one thread per filter quaternion walking the batch: beyond 128 rows the
// channels-last matrix-core kernel wins where it applies (64 -> 64 units, 1024 rows: 24 against 197 us for both gradients).
static bool dense_runs_small(const Problem& p, int pass) {
    if (!dense_is_small(p)) return false;
    Problem q;
    return !(pass == PHX_PASS_BWD_WEIGHTS && p.n > 128 && dense_as_channels_last(p, pass, q));
}

size_t phx_qdense_workspace_bytes(const phx_qdense_desc* desc, int pass) {
    if (desc && desc->algebra != PHX_QUATERNION) return algebra_dense_workspace_bytes(desc, pass);
    Problem p, q;
    if (problem_from_dense(desc, p) != PHX_OK) return 0;
    if (dense_runs_small(p, pass)) return 0;
    if (dense_as_channels_last(p, pass, q)) return pass == PHX_PASS_BWD_WEIGHTS ? workspace_for(q, pass) : nhwc_native_workspace(q, pass);
    return workspace_for(p, pass);
}

// The forward pass of a quaternion convolution (also walked "dry" by the packing session, see PackSession)
static int conv_fwd_quaternion(const phx_qconv_desc* desc, phx_stream_t stream, const void* x, const void* w,
                               const void* bias_or_null, void* y, void* workspace, size_t workspace_bytes) {
    const bool dry = g_pack.dry();
    Problem p;
    const int rc = problem_from_conv(desc, p);
    if (rc != PHX_OK) return rc;
    const bool direct = thin_groups(p, PHX_PASS_FWD);  // the vector-ALU kernels: groups of few channels, windows beyond the staging limit
    if (!direct && nhwc_native(p, PHX_PASS_FWD))
        return run_pwx_nhwc(p, MAP_FWD, static_cast<hipStream_t>(stream), x, w, p.has_bias ? bias_or_null : nullptr, y, workspace,
                            workspace_bytes);
    const GroupOffsets o(p);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (!direct && nhwc_window_native(p, PHX_PASS_FWD)) {
        g_window_cl = true;
        const int nrc = do_fwd(p, st, x, w, bias_or_null, y, dry ? nullptr : workspace, dry ? 0 : workspace_bytes);
        g_window_cl = false;
        return nrc;
    }
    const int merged = direct ? 0 : merged_groups(p, PHX_PASS_FWD);
    if (!direct && !merged && group_batchable(p, PHX_PASS_FWD)) {
        const GroupBatchScope batch(p);
        return do_fwd(p, st, x, w, bias_or_null, y, dry ? nullptr : workspace, dry ? 0 : workspace_bytes);
    }
    const ChannelsLast cl(p);
    if (dry) { workspace = nullptr; workspace_bytes = cl.bytes(); }
    else if (cl.bytes() > workspace_bytes || (cl.bytes() && !workspace)) return PHX_ERR_WORKSPACE;
    char* ws = static_cast<char*>(workspace);
    void* y_planes = y;
    if (p.nhwc && !dry) {
        cl.x_in(p, x, ws, st);
        x = ws;
        y_planes = ws + cl.x_bytes;
    }
    if (direct) {  // (no packed form: a packing session finds nothing to pack)
        if (g_pack.mode == PackSession::USE) return PHX_ERR_NOT_SUPPORTED;
        if (!dry)
            if (const int trc = run_thin(p, PHX_PASS_FWD, st, x, w, bias_or_null, y_planes, nullptr, 0)) return trc;
    } else if (merged) {
        if (const int mrc = run_merged(p, merged, PHX_PASS_FWD, st, x, w, bias_or_null, y_planes, ws ? ws + cl.bytes() : nullptr,
                                       workspace_bytes - cl.bytes()))
            return mrc;
    } else
    for (int g = 0; g < o.runs; ++g) {
        const int grc = do_fwd(p, st, o.at(x, g * o.x), o.at(w, g * o.w),
                               bias_or_null ? o.at(bias_or_null, g * o.b) : nullptr, o.at(y_planes, g * o.y),
                               ws ? ws + cl.bytes() : nullptr, workspace_bytes - cl.bytes());
        if (grc != PHX_OK) return grc;
    }
    if (p.nhwc && !dry) cl.y_out(p, y_planes, y, st);
    return PHX_OK;
}

int phx_qconv2d_fwd(const phx_qconv_desc* desc, phx_stream_t stream, const void* x, const void* w,
                    const void* bias_or_null, void* y, void* workspace, size_t workspace_bytes) {
    if (const int desc_rc = conv_desc_status(desc)) return desc_rc;
    if (const int init_rc = device_state(nullptr)) return init_rc;
    if (misaligned_workspace(workspace)) return PHX_ERR_INVALID_ARGUMENT;
    if (desc && desc->algebra != PHX_QUATERNION)
        return algebra_conv_pass(desc, PHX_PASS_FWD, stream, x, w, bias_or_null, y, workspace, workspace_bytes);
    return conv_fwd_quaternion(desc, stream, x, w, bias_or_null, y, workspace, workspace_bytes);
}

int phx_qconv2d_fwd_noalloc(const phx_qconv_desc* desc, phx_stream_t stream, const void* x, const void* w,
                            const void* bias_or_null, void* y) {
    if (const int desc_rc = conv_desc_status(desc)) return desc_rc;
    DeviceState* dev = nullptr;
    if (const int init_rc = device_state(&dev)) return init_rc;
    if (!dev->scratch_ptr) return PHX_ERR_RUNTIME;  // (the array's address could not be looked up on this device)
    if (phx_qconv2d_workspace_bytes(desc, PHX_PASS_FWD) > (size_t)PHX_NOALLOC_SCRATCH_BYTES) return PHX_ERR_SCRATCH_LIMIT;
    // the packed filters (and whatever else the forward pass stages) go to this device's copy of the scratch array
    return phx_qconv2d_fwd(desc, stream, x, w, bias_or_null, y, dev->scratch_ptr, PHX_NOALLOC_SCRATCH_BYTES);
}

static int conv_bwd_data_quaternion(const phx_qconv_desc* desc, phx_stream_t stream, const void* grad, const void* w, void* dx,
                                    void* workspace, size_t workspace_bytes) {
    const bool dry = g_pack.dry();
    Problem p;
    const int rc = problem_from_conv(desc, p);
    if (rc != PHX_OK) return rc;
    // the gradient with respect to a real-valued input has imaginary parts that are stored nowhere;
    // the reference refuses the request likewise (src/conv2d.hpp:394-398)
    if (p.real_input) return PHX_ERR_INVALID_ARGUMENT;
    const bool direct = thin_groups(p, PHX_PASS_BWD_DATA);
    if (!direct && nhwc_native(p, PHX_PASS_BWD_DATA))
        return run_pwx_nhwc(p, MAP_DGRAD, static_cast<hipStream_t>(stream), grad, w, nullptr, dx, workspace, workspace_bytes);
    const GroupOffsets o(p);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (!direct && nhwc_window_native(p, PHX_PASS_BWD_DATA)) {
        g_window_cl = true;
        const int nrc = do_bwd_data(p, st, grad, w, dx, dry ? nullptr : workspace, dry ? 0 : workspace_bytes);
        g_window_cl = false;
        return nrc;
    }
    const int merged = direct ? 0 : merged_groups(p, PHX_PASS_BWD_DATA);
    if (!direct && !merged && group_batchable(p, PHX_PASS_BWD_DATA)) {
        const GroupBatchScope batch(p);
        return do_bwd_data(p, st, grad, w, dx, dry ? nullptr : workspace, dry ? 0 : workspace_bytes);
    }
    const ChannelsLast cl(p);
    if (dry) { workspace = nullptr; workspace_bytes = cl.bytes(); }
    else if (cl.bytes() > workspace_bytes || (cl.bytes() && !workspace)) return PHX_ERR_WORKSPACE;
    char* ws = static_cast<char*>(workspace);
    void* dx_planes = dx;
    if (p.nhwc && !dry) {
        cl.y_in(p, grad, ws + cl.x_bytes, st);
        grad = ws + cl.x_bytes;
        dx_planes = ws;
    }
    if (direct) {
        if (g_pack.mode == PackSession::USE) return PHX_ERR_NOT_SUPPORTED;
        if (!dry)
            if (const int trc = run_thin(p, PHX_PASS_BWD_DATA, st, grad, w, nullptr, dx_planes, nullptr, 0)) return trc;
    } else if (merged) {
        if (const int mrc = run_merged(p, merged, PHX_PASS_BWD_DATA, st, grad, w, nullptr, dx_planes, ws ? ws + cl.bytes() : nullptr,
                                       workspace_bytes - cl.bytes()))
            return mrc;
    } else
    for (int g = 0; g < o.runs; ++g) {
        const int grc = do_bwd_data(p, st, o.at(grad, g * o.y), o.at(w, g * o.w), o.at(dx_planes, g * o.x),
                                    ws ? ws + cl.bytes() : nullptr, workspace_bytes - cl.bytes());
        if (grc != PHX_OK) return grc;
    }
    if (p.nhwc && !dry) cl.x_out(p, dx_planes, dx, st);
    return PHX_OK;
}

int phx_qconv2d_bwd_data(const phx_qconv_desc* desc, phx_stream_t stream, const void* grad, const void* w, void* dx,
                         void* workspace, size_t workspace_bytes) {
    if (const int desc_rc = conv_desc_status(desc)) return desc_rc;
    if (const int init_rc = device_state(nullptr)) return init_rc;
    if (misaligned_workspace(workspace)) return PHX_ERR_INVALID_ARGUMENT;
    if (desc && desc->algebra != PHX_QUATERNION)
        return algebra_conv_pass(desc, PHX_PASS_BWD_DATA, stream, grad, w, nullptr, dx, workspace, workspace_bytes);
    return conv_bwd_data_quaternion(desc, stream, grad, w, dx, workspace, workspace_bytes);
}

// ---- filters packed ahead of the passes ----
static bool prepack_pass_ok(int pass) { return pass == PHX_PASS_FWD || pass == PHX_PASS_BWD_DATA; }

static int walk_pass(const phx_qconv_desc* desc, int pass, phx_stream_t stream, const void* in, const void* w,
                     const void* bias, void* out, void* ws, size_t wsb) {
    return pass == PHX_PASS_FWD ? conv_fwd_quaternion(desc, stream, in, w, bias, out, ws, wsb)
                                : conv_bwd_data_quaternion(desc, stream, in, w, out, ws, wsb);
}

size_t phx_qconv2d_packed_filter_bytes(const phx_qconv_desc* desc, int pass) {
    if (!desc || desc->algebra != PHX_QUATERNION || !prepack_pass_ok(pass)) return 0;
    PackSessionScope scope(PackSession::SIZE, nullptr, 0, nullptr);
    if (walk_pass(desc, pass, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0) != PHX_OK) return 0;
    return g_pack.offset;
}

int phx_qconv2d_pack_filters(const phx_qconv_desc* desc, phx_stream_t stream, const void* w, void* packed_fwd,
                             size_t packed_fwd_bytes, void* packed_bwd_data, size_t packed_bwd_data_bytes) {
    if (const int desc_rc = conv_desc_status(desc)) return desc_rc;
    if (const int init_rc = device_state(nullptr)) return init_rc;
    if (!desc || desc->algebra != PHX_QUATERNION) return PHX_ERR_NOT_SUPPORTED;
    if (!w || (!packed_fwd && !packed_bwd_data)) return PHX_ERR_INVALID_ARGUMENT;
    if (misaligned_workspace(packed_fwd) || misaligned_workspace(packed_bwd_data)) return PHX_ERR_INVALID_ARGUMENT;
    g_pack.jobs.n = 0;
    void* const dst[2] = {packed_fwd, packed_bwd_data};
    const size_t cap[2] = {packed_fwd_bytes, packed_bwd_data_bytes};
    const int pass[2] = {PHX_PASS_FWD, PHX_PASS_BWD_DATA};
    for (int i = 0; i < 2; ++i) {
        if (!dst[i]) continue;
        PackSessionScope scope(PackSession::RECORD, dst[i], cap[i], static_cast<hipStream_t>(stream));
        const int rc = walk_pass(desc, pass[i], stream, nullptr, w, nullptr, nullptr, nullptr, 0);
        if (rc != PHX_OK) { g_pack.jobs.n = 0; return rc; }
        if (g_pack.offset == 0) { g_pack.jobs.n = 0; return PHX_ERR_NOT_SUPPORTED; }
    }
    g_pack.st = static_cast<hipStream_t>(stream);
    const int rc = flush_pack_jobs();  // both passes' images by one launch
    if (rc != PHX_OK) return rc;
    PHX_HIP(hipGetLastError());
    return PHX_OK;
}

int phx_qconv2d_fwd_prepacked(const phx_qconv_desc* desc, phx_stream_t stream, const void* x, const void* packed_fwd,
                              size_t packed_fwd_bytes, const void* bias_or_null, void* y, void* workspace,
                              size_t workspace_bytes) {
    if (const int desc_rc = conv_desc_status(desc)) return desc_rc;
    if (const int init_rc = device_state(nullptr)) return init_rc;
    if (!desc || desc->algebra != PHX_QUATERNION) return PHX_ERR_NOT_SUPPORTED;
    if (!packed_fwd || misaligned_workspace(workspace) || misaligned_workspace(packed_fwd)) return PHX_ERR_INVALID_ARGUMENT;
    PackSessionScope scope(PackSession::USE, const_cast<void*>(packed_fwd), packed_fwd_bytes, static_cast<hipStream_t>(stream));
    // (the filter argument of the walk only has to be non-null: nothing reads it)
    return conv_fwd_quaternion(desc, stream, x, packed_fwd, bias_or_null, y, workspace, workspace_bytes);
}

int phx_qconv2d_bwd_data_prepacked(const phx_qconv_desc* desc, phx_stream_t stream, const void* grad,
                                   const void* packed_bwd_data, size_t packed_bwd_data_bytes, void* dx, void* workspace,
                                   size_t workspace_bytes) {
    if (const int desc_rc = conv_desc_status(desc)) return desc_rc;
    if (const int init_rc = device_state(nullptr)) return init_rc;
    if (!desc || desc->algebra != PHX_QUATERNION) return PHX_ERR_NOT_SUPPORTED;
    if (!packed_bwd_data || misaligned_workspace(workspace) || misaligned_workspace(packed_bwd_data)) return PHX_ERR_INVALID_ARGUMENT;
    PackSessionScope scope(PackSession::USE, const_cast<void*>(packed_bwd_data), packed_bwd_data_bytes,
                           static_cast<hipStream_t>(stream));
    return conv_bwd_data_quaternion(desc, stream, grad, packed_bwd_data, dx, workspace, workspace_bytes);
}

int phx_qconv2d_bwd_data_add(const phx_qconv_desc* desc, phx_stream_t stream, const void* grad, const void* w,
                             const void* packed_bwd_data_or_null, size_t packed_bwd_data_bytes, const void* addend, void* dx,
                             void* workspace, size_t workspace_bytes) {
    if (const int desc_rc = conv_desc_status(desc)) return desc_rc;
    if (const int init_rc = device_state(nullptr)) return init_rc;
    if (!desc || desc->algebra != PHX_QUATERNION) return PHX_ERR_NOT_SUPPORTED;
    if (!addend || !dx || addend == dx) return PHX_ERR_INVALID_ARGUMENT;
    Problem p;
    if (const int prc = problem_from_conv(desc, p)) return prc;
    g_addend.ptr = addend; g_addend.dx = dx; g_addend.fused = false;
    const int rc = packed_bwd_data_or_null
                       ? phx_qconv2d_bwd_data_prepacked(desc, stream, grad, packed_bwd_data_or_null, packed_bwd_data_bytes, dx,
                                                        workspace, workspace_bytes)
                       : phx_qconv2d_bwd_data(desc, stream, grad, w, dx, workspace, workspace_bytes);
    const bool fused = g_addend.fused;
    g_addend = Addend{};
    if (rc != PHX_OK || fused || is_empty(p)) return rc;
    launch_add_inplace(p.dtype == PHX_F16, dx, addend, 4L * p.n * p.ci_mem * p.h * p.w, static_cast<hipStream_t>(stream));
    PHX_HIP(hipGetLastError());
    return PHX_OK;
}

int phx_qconv2d_bwd_weights(const phx_qconv_desc* desc, phx_stream_t stream, const void* x, const void* grad, void* dw,
                            void* workspace, size_t workspace_bytes) {
    if (const int desc_rc = conv_desc_status(desc)) return desc_rc;
    if (const int init_rc = device_state(nullptr)) return init_rc;
    if (misaligned_workspace(workspace)) return PHX_ERR_INVALID_ARGUMENT;
    if (desc && desc->algebra != PHX_QUATERNION)
        return algebra_conv_pass(desc, PHX_PASS_BWD_WEIGHTS, stream, x, grad, nullptr, dw, workspace, workspace_bytes);
    Problem p;
    const int rc = problem_from_conv(desc, p);
    if (rc != PHX_OK) return rc;
    const GroupOffsets o(p);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool direct = thin_groups(p, PHX_PASS_BWD_WEIGHTS);
    if (!direct && nhwc_wgrad_native(p)) {
        g_window_cl = true;
        const int nrc = do_bwd_weights(p, st, x, grad, dw, workspace, workspace_bytes);
        g_window_cl = false;
        return nrc;
    }
    const int merged = direct ? 0 : merged_groups(p, PHX_PASS_BWD_WEIGHTS);
    if (!direct && !merged && group_batchable(p, PHX_PASS_BWD_WEIGHTS)) {
        const GroupBatchScope batch(p);
        return do_bwd_weights(p, st, x, grad, dw, workspace, workspace_bytes);
    }
    const ChannelsLast cl(p);
    if (cl.bytes() > workspace_bytes || (cl.bytes() && !workspace)) return PHX_ERR_WORKSPACE;
    char* ws = static_cast<char*>(workspace);
    if (p.nhwc) {
        cl.x_in(p, x, ws, st);
        cl.y_in(p, grad, ws + cl.x_bytes, st);
        x = ws;
        grad = ws + cl.x_bytes;
    }
    if (merged)
        return run_merged(p, merged, PHX_PASS_BWD_WEIGHTS, st, x, grad, nullptr, dw, ws ? ws + cl.bytes() : nullptr,
                          workspace_bytes - cl.bytes());
    if (direct)
        return run_thin(p, PHX_PASS_BWD_WEIGHTS, st, x, grad, nullptr, dw, ws ? ws + cl.bytes() : nullptr, workspace_bytes - cl.bytes());
    for (int g = 0; g < o.runs; ++g) {
        const int grc = do_bwd_weights(p, st, o.at(x, g * o.x), o.at(grad, g * o.y), o.at(dw, g * o.w),
                                       ws ? ws + cl.bytes() : nullptr, workspace_bytes - cl.bytes());
        if (grc != PHX_OK) return grc;
    }
    return PHX_OK;
}

int phx_qdense_fwd(const phx_qdense_desc* desc, phx_stream_t stream, const void* x, const void* w,
                   const void* bias_or_null, void* y, void* workspace, size_t workspace_bytes) {
    if (const int desc_rc = dense_desc_status(desc)) return desc_rc;
    if (const int init_rc = device_state(nullptr)) return init_rc;
    if (misaligned_workspace(workspace)) return PHX_ERR_INVALID_ARGUMENT;
    if (desc && desc->algebra != PHX_QUATERNION)
        return algebra_dense_pass(desc, PHX_PASS_FWD, stream, x, w, bias_or_null, y, workspace, workspace_bytes);
    Problem p;
    const int rc = problem_from_dense(desc, p);
    if (rc != PHX_OK) return rc;
    if (dense_runs_small(p, PHX_PASS_FWD)) return is_empty(p) ? PHX_OK : run_dense_small(p, PHX_PASS_FWD, static_cast<hipStream_t>(stream), x, w, bias_or_null, y);
    Problem q;
    if (dense_as_channels_last(p, PHX_PASS_FWD, q))
        return run_pwx_nhwc(q, MAP_FWD, static_cast<hipStream_t>(stream), x, w, q.has_bias ? bias_or_null : nullptr, y, workspace, workspace_bytes);
    return do_fwd(p, static_cast<hipStream_t>(stream), x, w, bias_or_null, y, workspace, workspace_bytes);
}

int phx_qdense_bwd_data(const phx_qdense_desc* desc, phx_stream_t stream, const void* grad, const void* w, void* dx,
                        void* workspace, size_t workspace_bytes) {
    if (const int desc_rc = dense_desc_status(desc)) return desc_rc;
    if (const int init_rc = device_state(nullptr)) return init_rc;
    if (misaligned_workspace(workspace)) return PHX_ERR_INVALID_ARGUMENT;
    if (desc && desc->algebra != PHX_QUATERNION)
        return algebra_dense_pass(desc, PHX_PASS_BWD_DATA, stream, grad, w, nullptr, dx, workspace, workspace_bytes);
    Problem p;
    const int rc = problem_from_dense(desc, p);
    if (rc != PHX_OK) return rc;
    if (dense_runs_small(p, PHX_PASS_BWD_DATA)) return is_empty(p) ? PHX_OK : run_dense_small(p, PHX_PASS_BWD_DATA, static_cast<hipStream_t>(stream), grad, w, nullptr, dx);
    Problem q;
    if (dense_as_channels_last(p, PHX_PASS_BWD_DATA, q))
        return run_pwx_nhwc(q, MAP_DGRAD, static_cast<hipStream_t>(stream), grad, w, nullptr, dx, workspace, workspace_bytes);
    return do_bwd_data(p, static_cast<hipStream_t>(stream), grad, w, dx, workspace, workspace_bytes);
}

int phx_qdense_bwd_weights(const phx_qdense_desc* desc, phx_stream_t stream, const void* x, const void* grad, void* dw,
                           void* workspace, size_t workspace_bytes) {
    if (const int desc_rc = dense_desc_status(desc)) return desc_rc;
    if (const int init_rc = device_state(nullptr)) return init_rc;
    if (misaligned_workspace(workspace)) return PHX_ERR_INVALID_ARGUMENT;
    if (desc && desc->algebra != PHX_QUATERNION)
        return algebra_dense_pass(desc, PHX_PASS_BWD_WEIGHTS, stream, x, grad, nullptr, dw, workspace, workspace_bytes);
    Problem p;
    const int rc = problem_from_dense(desc, p);
    if (rc != PHX_OK) return rc;
    if (dense_runs_small(p, PHX_PASS_BWD_WEIGHTS)) return run_dense_small(p, PHX_PASS_BWD_WEIGHTS, static_cast<hipStream_t>(stream), x, grad, nullptr, dw);
    Problem q;
    if (dense_as_channels_last(p, PHX_PASS_BWD_WEIGHTS, q)) {
        g_window_cl = true;
        const int qrc = do_bwd_weights(q, static_cast<hipStream_t>(stream), x, grad, dw, workspace, workspace_bytes);
        g_window_cl = false;
        return qrc;
    }
    return do_bwd_weights(p, static_cast<hipStream_t>(stream), x, grad, dw, workspace, workspace_bytes);
}

int phx_device_count(int32_t* count) {
    int c = 0;
    if (hipGetDeviceCount(&c) != hipSuccess) { (void)hipGetLastError(); c = 0; }
    if (count) *count = c;
    return PHX_OK;
}

int phx_device_malloc(void** ptr, size_t bytes) {
    if (!ptr) return PHX_ERR_INVALID_ARGUMENT;
    *ptr = nullptr;
    if (bytes == 0) return PHX_OK;
    PHX_HIP(hipMalloc(ptr, bytes));
    return PHX_OK;
}

int phx_device_free(void* ptr) {
    if (ptr) PHX_HIP(hipFree(ptr));
    return PHX_OK;
}

int phx_memcpy_h2d(void* dst, const void* src, size_t bytes, phx_stream_t stream) {
    if (bytes == 0) return PHX_OK;
    PHX_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, static_cast<hipStream_t>(stream)));
    PHX_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    return PHX_OK;
}

int phx_memcpy_d2h(void* dst, const void* src, size_t bytes, phx_stream_t stream) {
    if (bytes == 0) return PHX_OK;
    PHX_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream)));
    PHX_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    return PHX_OK;
}

int phx_memset_zero(void* dst, size_t bytes, phx_stream_t stream) {
    if (bytes == 0) return PHX_OK;
    launch_fill_zero(dst, bytes, static_cast<hipStream_t>(stream));
    PHX_HIP(hipGetLastError());
    return PHX_OK;
}

int phx_stream_create(phx_stream_t* stream) {
    if (!stream) return PHX_ERR_INVALID_ARGUMENT;
    hipStream_t s;
    PHX_HIP(hipStreamCreate(&s));
    *stream = s;
    return PHX_OK;
}

int phx_stream_destroy(phx_stream_t stream) {
    if (stream) PHX_HIP(hipStreamDestroy(static_cast<hipStream_t>(stream)));
    return PHX_OK;
}

int phx_stream_synchronize(phx_stream_t stream) {
    PHX_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    return PHX_OK;
}

}  // extern "C"
