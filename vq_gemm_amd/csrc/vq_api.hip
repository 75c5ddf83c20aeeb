// C ABI of libvqgemm.so: argument validation and kernel selection.  No torch types here;
// the torch extension and the tests both call these entry points.
#include "../../include/vq_gemm.h"
#include "vq_common.h"

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <limits.h>
#include <map>
#include <mutex>
#include <string>
#include <utility>

namespace vq {

int device_cu_count()
{
    constexpr int kMaxDev = 64;
    static std::atomic<int> cache[kMaxDev];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDev) return 256;
    int v = cache[dev].load(std::memory_order_relaxed);
    if (v > 0) return v;
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    cache[dev].store(cus, std::memory_order_relaxed);
    return cus;
}

hipError_t ensure_dynamic_lds(const void *kernel, size_t bytes)
{
    if (bytes <= 48 * 1024) return hipSuccess;  // within the default limit
    static std::mutex mu;
    static std::map<std::pair<int, const void *>, size_t> granted;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    std::lock_guard<std::mutex> lock(mu);
    size_t &g = granted[{dev, kernel}];
    if (bytes <= g) return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e == hipSuccess) g = bytes;
    return e;
}

namespace {

struct TuningEntry {
    const char *name;
    double Tuning::*field;
};
const TuningEntry kTuningEntries[] = {
    {"prefill_tile_fixed_us", &Tuning::prefill_tile_fixed_us},
    {"prefill_stage_us_256x256", &Tuning::prefill_stage_us_256x256},
    {"prefill_stage_us_256x128", &Tuning::prefill_stage_us_256x128},
    {"prefill_full_device_factor", &Tuning::prefill_full_device_factor},
    {"prefill_small_tile_fixed_us", &Tuning::prefill_small_tile_fixed_us},
    {"prefill_small_stage_us_idle", &Tuning::prefill_small_stage_us_idle},
    {"prefill_small_stage_us_busy", &Tuning::prefill_small_stage_us_busy},
    {"decode_prologue_us", &Tuning::decode_prologue_us},
    {"decode_prologue_shared_cu_us", &Tuning::decode_prologue_shared_cu_us},
    {"decode_tile_us", &Tuning::decode_tile_us},
    {"decode_tile_chunked_us", &Tuning::decode_tile_chunked_us},
    {"decode_pass_change_us", &Tuning::decode_pass_change_us},
    {"gemv_max_tiles_per_cu", &Tuning::gemv_max_tiles_per_cu},
    {"gemv_max_k", &Tuning::gemv_max_k},
    {"gemv_wide_min_rows_per_wave", &Tuning::gemv_wide_min_rows_per_wave},
    {"gemv_wide_max_m", &Tuning::gemv_wide_max_m},
    {"gemv_wide_two_rows_max_runs", &Tuning::gemv_wide_two_rows_max_runs},
    {"gemv_wide_two_rows_max_runs_long_k", &Tuning::gemv_wide_two_rows_max_runs_long_k},
    {"gemv_wide_plain_table_max_runs", &Tuning::gemv_wide_plain_table_max_runs},
    {"gemv_wide_single_rows_max", &Tuning::gemv_wide_single_rows_max},
    {"gemv_wide_rows_per_group", &Tuning::gemv_wide_rows_per_group},
    {"gemv_wide_groups_in_flight", &Tuning::gemv_wide_groups_in_flight},
    {"gemv_wide_rows_per_group_long_k", &Tuning::gemv_wide_rows_per_group_long_k},
    {"gemv_wide_groups_in_flight_long_k", &Tuning::gemv_wide_groups_in_flight_long_k},
    {"gemv_wide_rotate_priority", &Tuning::gemv_wide_rotate_priority},
    {"gemv_wide_min_units_share", &Tuning::gemv_wide_min_units_share},
    {"decode_replicated_table_min_tiles", &Tuning::decode_replicated_table_min_tiles},
    {"decode_stream_min_k", &Tuning::decode_stream_min_k},
    {"decode_stream_min_k_few_rows", &Tuning::decode_stream_min_k_few_rows},
    {"decode_stream_min_m", &Tuning::decode_stream_min_m},
    {"decode_stream_max_m", &Tuning::decode_stream_max_m},
    {"decode_stream_max_groups_per_unit", &Tuning::decode_stream_max_groups_per_unit},
    {"decode_stream_replicated_min_gathers", &Tuning::decode_stream_replicated_min_gathers},
    {"tail_split_margin", &Tuning::tail_split_margin},
    {"splitk_fixed_us", &Tuning::splitk_fixed_us},
    {"splitk_us_per_partial_mb", &Tuning::splitk_us_per_partial_mb},
    {"splitk_force_splits", &Tuning::splitk_force_splits},
    {"splitk_validate_fences", &Tuning::splitk_validate_fences},
};
constexpr int kTuningCount = (int)(sizeof(kTuningEntries) / sizeof(kTuningEntries[0]));

std::mutex g_tuning_mu;
Tuning g_tuning;             // written under the mutex; read without it (plain doubles, set before the launches that use them)
std::atomic<bool> g_tuning_file_read{false};  // (acquire/release: a reader that sees true also sees what the file set)

const TuningEntry *find_tuning(const char *name)
{
    if (!name) return nullptr;
    for (const TuningEntry &e : kTuningEntries)
        if (std::strcmp(e.name, name) == 0) return &e;
    return nullptr;
}

// A flat JSON object of numbers, {"name": value, ...}: names this library does not know are skipped, and so
// is everything that is no number (a "device" string, for instance).  Returns how many constants were set.
int read_tuning_file(const char *path)
{
    FILE *f = std::fopen(path, "rb");
    if (!f) return -1;
    std::string text;
    char buf[4096];
    size_t n;
    while ((n = std::fread(buf, 1, sizeof(buf), f)) > 0) text.append(buf, n);
    std::fclose(f);
    int set = 0;
    size_t pos = 0;
    while ((pos = text.find('"', pos)) != std::string::npos) {
        const size_t end = text.find('"', pos + 1);
        if (end == std::string::npos) break;
        const std::string key = text.substr(pos + 1, end - pos - 1);
        size_t q = end + 1;
        while (q < text.size() && (text[q] == ' ' || text[q] == '\t' || text[q] == '\n' || text[q] == '\r')) q++;
        pos = end + 1;
        if (q >= text.size() || text[q] != ':') continue;   // a string value, not a key
        q++;
        while (q < text.size() && (text[q] == ' ' || text[q] == '\t' || text[q] == '\n' || text[q] == '\r')) q++;
        char *stop = nullptr;
        const double v = std::strtod(text.c_str() + q, &stop);
        if (stop == text.c_str() + q) { pos = q; continue; }  // no number behind the key
        pos = (size_t)(stop - text.c_str());
        const TuningEntry *e = find_tuning(key.c_str());
        if (e && v == v && v >= 0.0 && v < 1e9) {
            g_tuning.*(e->field) = v;
            set++;
        }
    }
    return set;
}

bool aligned(const void *p, uintptr_t a) { return ((uintptr_t)p & (a - 1)) == 0; }

// Whether the automatic choice takes the fused geometry-A kernel: at every height (a short X
// leaves its 128-row tile mostly padding, and the kernel is still an order of magnitude ahead of the
// scalar one).  Its 4-byte gathers keep the LDS busier than the matrix cores, so once there is more
// than one round of tiles the two-pass route is faster - when the caller brings the scratch for it.
bool fused_a_preferred(const ProblemA &p, bool has_workspace)
{
    if (p.M < 1 || !fused_a_supports(p)) return false;
    if (!has_workspace) return true;
    const int64_t tiles = (int64_t)((p.M + 255) / 256) * ((2 * p.Nc + 127) / 128);
    return tiles <= device_cu_count();
}

int check_b(int64_t M, int64_t K, int64_t N, int32_t vec, int32_t entries, int32_t n_codebooks, int32_t code_bits)
{
    if (M < 0 || K < 0 || N < 0 || M > INT_MAX / 2 || K > INT_MAX / 2 || N > INT_MAX / 2) return VQGEMM_E_SHAPE;
    if (vec < 1 || vec > 4096 || entries < 1 || n_codebooks < 1) return VQGEMM_E_SHAPE;
    if (code_bits != 8 && code_bits != 16) return VQGEMM_E_CODEBITS;
    if ((int64_t)entries > ((int64_t)1 << code_bits)) return VQGEMM_E_CODEBITS;
    if (K % vec != 0) return VQGEMM_E_SHAPE;
    if (N % n_codebooks != 0) return VQGEMM_E_SHAPE;
    return VQGEMM_OK;
}

ProblemB make_b(const void *x, const void *codes, const void *codebook, void *y, int64_t M, int64_t K, int64_t N,
                int32_t vec, int32_t entries, int32_t n_codebooks, int32_t code_bits)
{
    ProblemB p;
    p.x = static_cast<const half_t *>(x);
    p.codes = codes;
    p.cb = static_cast<const half_t *>(codebook);
    p.y = static_cast<half_t *>(y);
    p.bias = nullptr;
    p.M = (int)M; p.K = (int)K; p.N = (int)N;
    p.vec = vec; p.entries = entries; p.n_codebooks = n_codebooks; p.code_bits = code_bits;
    p.rows_per_cb = N > 0 ? (int)(N / n_codebooks) : 1;
    if (p.rows_per_cb < 1) p.rows_per_cb = 1;
    p.packed = false;
    p.gated = false;
    return p;
}

int select_b(const ProblemB &p, bool all_aligned16)
{
    if (p.K == 0 || !all_aligned16) return VQGEMM_VARIANT_GENERIC;
    if (decode_gemv_wide_preferred(p)) return VQGEMM_VARIANT_DECODE_GEMV;  // (also shapes the K-sliced kernels refuse)
    const bool prefill_ok = prefill_supports(p);
    if (decode_supports(p) && (!prefill_ok || decode_preferred(p)))
        return decode_gemv_preferred(p) ? VQGEMM_VARIANT_DECODE_GEMV : VQGEMM_VARIANT_DECODE;
    if (prefill_ok) return VQGEMM_VARIANT_PREFILL;
    return VQGEMM_VARIANT_GENERIC;
}

}  // namespace

const Tuning &tuning()
{
    // the file named by VQGEMM_TUNING_FILE is read once, at the first question
    if (!g_tuning_file_read.load(std::memory_order_acquire)) {
        std::lock_guard<std::mutex> lock(g_tuning_mu);
        if (!g_tuning_file_read.load(std::memory_order_relaxed)) {
            const char *path = std::getenv("VQGEMM_TUNING_FILE");
            if (path && path[0]) read_tuning_file(path);
            g_tuning_file_read.store(true, std::memory_order_release);
        }
    }
    return g_tuning;
}

}  // namespace vq

using namespace vq;

extern "C" {

int vqgemm_version(void) { return 200; }

int vqgemm_tuning_count(void) { return kTuningCount; }

const char *vqgemm_tuning_name(int index) { return index >= 0 && index < kTuningCount ? kTuningEntries[index].name : nullptr; }

int vqgemm_tuning_get(const char *name, double *value)
{
    const TuningEntry *e = find_tuning(name);
    if (!e) return VQGEMM_E_VARIANT;
    if (!value) return VQGEMM_E_NULL;
    *value = tuning().*(e->field);
    return VQGEMM_OK;
}

int vqgemm_tuning_set(const char *name, double value)
{
    const TuningEntry *e = find_tuning(name);
    if (!e) return VQGEMM_E_VARIANT;
    if (!(value >= 0.0) || value >= 1e9) return VQGEMM_E_SHAPE;
    (void)tuning();  // (a file is read before, not after, an explicit setting)
    std::lock_guard<std::mutex> lock(g_tuning_mu);
    g_tuning.*(e->field) = value;
    return VQGEMM_OK;
}

int vqgemm_tuning_load(const char *path)
{
    if (!path) return VQGEMM_E_NULL;
    (void)tuning();
    std::lock_guard<std::mutex> lock(g_tuning_mu);
    const int n = read_tuning_file(path);
    return n < 0 ? VQGEMM_E_NULL : n;
}

const char *vqgemm_error_string(int code)
{
    switch (code) {
    case VQGEMM_OK: return "success";
    case VQGEMM_E_NULL: return "a required pointer is NULL";
    case VQGEMM_E_SHAPE: return "invalid shape (negative or too large size, K % vec != 0, N % n_codebooks != 0, ...)";
    case VQGEMM_E_CODEBITS: return "code_bits must be 8 or 16 and entries <= 2^code_bits";
    case VQGEMM_E_VARIANT: return "unknown kernel variant, or the variant cannot serve this shape";
    case VQGEMM_E_ALIGN: return "pointer not aligned as the selected kernel requires";
    case VQGEMM_E_SCRATCH: return "the problem needs more scratch than the library's fixed device array, or the workspace passed with its size, holds";
    default: break;
    }
    if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
    return "unknown vqgemm error";
}

int vqgemm_select_variant_b(int64_t M, int64_t K, int64_t N, int32_t vec, int32_t entries, int32_t n_codebooks,
                            int32_t code_bits)
{
    const int rc = check_b(M, K, N, vec, entries, n_codebooks, code_bits);
    if (rc != VQGEMM_OK) return rc;
    const ProblemB p = make_b(nullptr, nullptr, nullptr, nullptr, M, K, N, vec, entries, n_codebooks, code_bits);
    return select_b(p, true);
}

int vqgemm_e2e_gemm_b_bias(const void *x, const void *codes, const void *codebook, const void *bias, void *y,
                           int64_t M, int64_t K, int64_t N, int32_t vec, int32_t entries, int32_t n_codebooks,
                           int32_t code_bits, int32_t variant, void *workspace, void *stream)
{
    int rc = check_b(M, K, N, vec, entries, n_codebooks, code_bits);
    if (rc != VQGEMM_OK) return rc;
    if (variant < VQGEMM_VARIANT_AUTO || variant > VQGEMM_VARIANT_DECODE_GEMV) return VQGEMM_E_VARIANT;
    if (M == 0 || N == 0) return VQGEMM_OK;
    if (!y || !codebook || (K > 0 && (!x || !codes))) return VQGEMM_E_NULL;
    const uintptr_t code_align = code_bits / 8;
    if (!aligned(x, 2) || !aligned(y, 2) || !aligned(codebook, 2) || !aligned(codes, code_align)) return VQGEMM_E_ALIGN;
    if (!aligned(bias, 2)) return VQGEMM_E_ALIGN;
    // the tiled kernels read four bias values at a time
    const bool a16 = aligned(x, 16) && aligned(y, 16) && aligned(codebook, 16) && aligned(codes, 16) && aligned(bias, 8);
    ProblemB p = make_b(x, codes, codebook, y, M, K, N, vec, entries, n_codebooks, code_bits);
    p.bias = static_cast<const half_t *>(bias);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (variant == VQGEMM_VARIANT_AUTO) variant = select_b(p, a16);
    hipError_t e = hipSuccess;
    switch (variant) {
    case VQGEMM_VARIANT_GENERIC:
        e = launch_generic_b(p, s);
        break;
    case VQGEMM_VARIANT_DECODE:
        if (!a16) return VQGEMM_E_ALIGN;
        if (K == 0 || !decode_supports(p)) return VQGEMM_E_VARIANT;
        e = launch_decode_b(p, s);
        break;
    case VQGEMM_VARIANT_DECODE_GEMV:
        if (!a16) return VQGEMM_E_ALIGN;
        if (K == 0 || !decode_gemv_supports(p)) return VQGEMM_E_VARIANT;
        e = launch_decode_gemv(p, s);
        break;
    case VQGEMM_VARIANT_DECODE_PACKED:
        if (!a16) return VQGEMM_E_ALIGN;
        p.packed = true;
        if (K == 0 || !decode_packed_supports(p)) return VQGEMM_E_VARIANT;
        e = launch_decode_b(p, s);
        break;
    case VQGEMM_VARIANT_PREFILL:
        if (!a16) return VQGEMM_E_ALIGN;
        if (K == 0 || !prefill_supports(p)) return VQGEMM_E_VARIANT;
        e = launch_prefill_b(p, s);
        break;
    case VQGEMM_VARIANT_PREFILL_NARROW:
        if (!a16) return VQGEMM_E_ALIGN;
        if (K == 0 || !prefill_narrow_supports(p)) return VQGEMM_E_VARIANT;
        e = launch_prefill_b(p, s, 2);
        break;
    case VQGEMM_VARIANT_PREFILL_SMALL:
        if (!a16) return VQGEMM_E_ALIGN;
        if (K == 0 || !prefill_small_supports(p)) return VQGEMM_E_VARIANT;
        e = launch_prefill_small_b(p, s);
        break;
    case VQGEMM_VARIANT_TWOPASS:
        if (bias) return VQGEMM_E_VARIANT;  // the plain GEMM of the two-pass route has no bias input
        if (!workspace) return VQGEMM_E_NULL;
        if (!aligned(workspace, 16)) return VQGEMM_E_ALIGN;
        e = launch_dequant_b(p, static_cast<half_t *>(workspace), s);
        if (e == hipSuccess)
            e = launch_gemm_nt(p.x, static_cast<const half_t *>(workspace), p.y, p.M, p.K, p.N, s);
        break;
    default:
        return VQGEMM_E_VARIANT;
    }
    return static_cast<int>(e);
}

namespace {

// Split K with the cost model's number of slices when that is expected to beat what the automatic choice would
// launch otherwise by a margin (and then at least two slices); 0: do not split.
int splitk_auto(const ProblemB &p, bool all_aligned16, double *t_best = nullptr, int *plain_variant = nullptr)
{
    if (t_best) *t_best = 1e30;
    if (p.K == 0 || !all_aligned16 || p.gated) return 0;
    const int plain = select_b(p, all_aligned16);
    if (plain_variant) *plain_variant = plain;
    double t_plain;
    if (plain == VQGEMM_VARIANT_PREFILL) t_plain = prefill_cost_us(p);
    else if (plain == VQGEMM_VARIANT_DECODE) t_plain = decode_cost_us(p);
    else return 0;
    if (t_plain >= 1e29) return 0;  // (short X: the decode path is taken without a comparison, and stays)
    double t_split = 1e30;
    const int sp = prefill_splitk_choice(p, &t_split, 2);
    const bool take = sp >= 2 && t_split < 0.9 * t_plain;
    if (t_best) *t_best = take ? t_split : t_plain;
    return take ? sp : 0;
}

// What the automatic choice does with a workspace: nothing, K split over every 128x128 tile (sp slices), or whole rounds
// of large tiles with the left-over columns in 128x128 tiles and K split there (tail) - whichever the cost models
// expect to be fastest by a margin.
struct WorkspaceChoice {
    int sp;
    TailSplitPlan tail;
    size_t bytes;
};
WorkspaceChoice workspace_auto(const ProblemB &p, bool all_aligned16)
{
    WorkspaceChoice c = {0, {false, 0, 0, 0, 1e30, 0}, 0};
    double t_best = 1e30;
    int plain = 0;
    c.sp = splitk_auto(p, all_aligned16, &t_best, &plain);
    if (c.sp >= 2) c.bytes = prefill_splitk_workspace_bytes(p, c.sp);
    if (plain == VQGEMM_VARIANT_PREFILL && t_best < 1e29) {
        const TailSplitPlan tail = prefill_tail_split_plan(p);
        // (a margin of 1000 and more: wherever the plan exists - for measurements and tests)
        const double margin = tuning().tail_split_margin;
        if (tail.ok && (margin >= 1e3 || tail.cost_us < margin * t_best)) {
            c.sp = 0;
            c.tail = tail;
            c.bytes = tail.workspace_bytes;
        }
    }
    return c;
}

}  // namespace

int64_t vqgemm_workspace_bytes_b(int64_t M, int64_t K, int64_t N, int32_t vec, int32_t entries, int32_t n_codebooks,
                                 int32_t code_bits, int32_t variant)
{
    const int rc = check_b(M, K, N, vec, entries, n_codebooks, code_bits);
    if (rc != VQGEMM_OK) return rc;
    if (M == 0 || N == 0 || K == 0) return 0;
    const ProblemB p = make_b(nullptr, nullptr, nullptr, nullptr, M, K, N, vec, entries, n_codebooks, code_bits);
    if (variant == VQGEMM_VARIANT_TWOPASS) return N * K * 2;
    if (variant == VQGEMM_VARIANT_AUTO) return (int64_t)workspace_auto(p, true).bytes;
    int sp = 0;
    if (variant == VQGEMM_VARIANT_PREFILL_SPLITK) sp = prefill_splitk_choice(p, nullptr, 2);
    return sp >= 2 ? (int64_t)prefill_splitk_workspace_bytes(p, sp) : 0;
}

int vqgemm_e2e_gemm_b_ws(const void *x, const void *codes, const void *codebook, const void *bias, void *y, int64_t M,
                         int64_t K, int64_t N, int32_t vec, int32_t entries, int32_t n_codebooks, int32_t code_bits,
                         int32_t variant, void *workspace, int64_t workspace_bytes, void *stream)
{
    if (workspace_bytes < 0 || (workspace_bytes > 0 && !workspace)) return VQGEMM_E_NULL;
    if (variant == VQGEMM_VARIANT_TWOPASS) {
        if (workspace_bytes < N * K * 2) return VQGEMM_E_SCRATCH;
        return vqgemm_e2e_gemm_b_bias(x, codes, codebook, bias, y, M, K, N, vec, entries, n_codebooks, code_bits, variant, workspace, stream);
    }
    if (variant != VQGEMM_VARIANT_AUTO && variant != VQGEMM_VARIANT_PREFILL_SPLITK)
        return vqgemm_e2e_gemm_b_bias(x, codes, codebook, bias, y, M, K, N, vec, entries, n_codebooks, code_bits, variant, nullptr, stream);
    int rc = check_b(M, K, N, vec, entries, n_codebooks, code_bits);
    if (rc != VQGEMM_OK) return rc;
    if (M == 0 || N == 0) return VQGEMM_OK;
    if (!y || !codebook || (K > 0 && (!x || !codes))) return VQGEMM_E_NULL;
    const bool a16 = aligned(x, 16) && aligned(y, 16) && aligned(codebook, 16) && aligned(codes, 16) && aligned(bias, 8) &&
                     aligned(workspace, 256);
    ProblemB p = make_b(x, codes, codebook, y, M, K, N, vec, entries, n_codebooks, code_bits);
    p.bias = static_cast<const half_t *>(bias);
    int sp;
    if (variant == VQGEMM_VARIANT_PREFILL_SPLITK) {
        if (!a16) return VQGEMM_E_ALIGN;
        sp = K > 0 ? prefill_splitk_choice(p, nullptr, 2) : 0;
        if (sp < 2) return VQGEMM_E_VARIANT;
        if ((int64_t)prefill_splitk_workspace_bytes(p, sp) > workspace_bytes) return VQGEMM_E_SCRATCH;
    } else {
        const WorkspaceChoice c = workspace_auto(p, a16);
        if (c.tail.ok && (int64_t)c.bytes <= workspace_bytes)
            return static_cast<int>(launch_prefill_tail_split(p, c.tail, static_cast<hipStream_t>(stream), workspace));
        sp = c.tail.ok ? splitk_auto(p, a16) : c.sp;
        // (a workspace that is too small is not an error for the automatic choice: it does without)
        if (sp < 2 || (int64_t)prefill_splitk_workspace_bytes(p, sp) > workspace_bytes)
            return vqgemm_e2e_gemm_b_bias(x, codes, codebook, bias, y, M, K, N, vec, entries, n_codebooks, code_bits, VQGEMM_VARIANT_AUTO,
                                          nullptr, stream);
    }
    return static_cast<int>(launch_prefill_small_b(p, static_cast<hipStream_t>(stream), sp, workspace));
}

int vqgemm_e2e_gemm_b_gated(const void *x, const void *codes, const void *codebook, const void *bias, void *y, int64_t M,
                            int64_t K, int64_t N, int32_t vec, int32_t entries, int32_t n_codebooks, int32_t code_bits,
                            int32_t variant, void *workspace, void *stream)
{
    int rc = check_b(M, K, N, vec, entries, n_codebooks, code_bits);
    if (rc != VQGEMM_OK) return rc;
    if (N % 32 != 0) return VQGEMM_E_SHAPE;  // whole pairs of 16 gate rows and 16 up rows
    if (M == 0 || N == 0) return VQGEMM_OK;
    if (!y || !codebook || (K > 0 && (!x || !codes))) return VQGEMM_E_NULL;
    const uintptr_t code_align = code_bits / 8;
    if (!aligned(x, 2) || !aligned(y, 2) || !aligned(codebook, 2) || !aligned(codes, code_align) || !aligned(bias, 2) ||
        !aligned(workspace, 2))
        return VQGEMM_E_ALIGN;
    const bool a16 = aligned(x, 16) && aligned(y, 16) && aligned(codebook, 16) && aligned(codes, 16) && aligned(bias, 8) &&
                     aligned(workspace, 16);
    ProblemB p = make_b(x, codes, codebook, y, M, K, N, vec, entries, n_codebooks, code_bits);
    p.bias = static_cast<const half_t *>(bias);
    p.gated = true;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // the plain product of the same shape, for the kernels without a gated epilogue (into the workspace)
    ProblemB plain = p;
    plain.gated = false;
    plain.y = static_cast<half_t *>(workspace);
    if (variant == VQGEMM_VARIANT_AUTO) {
        if (K == 0 || !a16) variant = VQGEMM_VARIANT_GENERIC;
        else if (decode_gemv_wide_preferred(p)) variant = VQGEMM_VARIANT_DECODE_GEMV;
        else {
            // What the plain product would run on decides: every tiled kernel carries the gated epilogue itself (the
            // GEMV kernels and the K-sliced decode kernels want whole groups of 32 interleaved rows per codebook
            // resp. per matrix; where one of them refuses, the next in line takes the shape).
            const int plain_variant = select_b(plain, true);
            if (plain_variant == VQGEMM_VARIANT_DECODE_GEMV && decode_gemv_supports(p)) variant = VQGEMM_VARIANT_DECODE_GEMV;
            else if ((plain_variant == VQGEMM_VARIANT_DECODE || plain_variant == VQGEMM_VARIANT_DECODE_GEMV) && decode_gated_supports(p))
                variant = VQGEMM_VARIANT_DECODE;
            else if (prefill_supports(plain)) variant = VQGEMM_VARIANT_PREFILL;
            else variant = VQGEMM_VARIANT_GENERIC;
        }
    }
    hipError_t e = hipSuccess;
    switch (variant) {
    case VQGEMM_VARIANT_GENERIC:
        e = launch_generic_b(p, s);
        break;
    case VQGEMM_VARIANT_DECODE_GEMV:
        if (!a16) return VQGEMM_E_ALIGN;
        if (K == 0 || !decode_gemv_supports(p)) return VQGEMM_E_VARIANT;
        e = launch_decode_gemv(p, s);
        break;
    case VQGEMM_VARIANT_DECODE:
        if (!a16) return VQGEMM_E_ALIGN;
        if (K == 0 || !decode_gated_supports(p)) return VQGEMM_E_VARIANT;
        e = launch_decode_b(p, s);
        break;
    case VQGEMM_VARIANT_PREFILL:
        if (!a16) return VQGEMM_E_ALIGN;
        if (K == 0 || !prefill_supports(plain)) return VQGEMM_E_VARIANT;
        e = launch_prefill_b(p, s);
        break;
    case VQGEMM_VARIANT_PREFILL_NARROW:
        if (!a16) return VQGEMM_E_ALIGN;
        if (K == 0 || !prefill_narrow_supports(plain)) return VQGEMM_E_VARIANT;
        e = launch_prefill_b(p, s, 2);
        break;
    case VQGEMM_VARIANT_PREFILL_SMALL:
        if (!a16) return VQGEMM_E_ALIGN;
        if (K == 0 || !prefill_small_supports(plain)) return VQGEMM_E_VARIANT;
        e = launch_prefill_small_b(p, s);
        break;
    case VQGEMM_VARIANT_TWOPASS: {
        // (here: the fused product as the automatic choice runs it, then the element-wise pass)
        if (!workspace) return VQGEMM_E_NULL;
        rc = vqgemm_e2e_gemm_b_bias(x, codes, codebook, bias, workspace, M, K, N, vec, entries, n_codebooks, code_bits,
                                    VQGEMM_VARIANT_AUTO, nullptr, stream);
        if (rc != VQGEMM_OK) return rc;
        e = launch_silu_mul(static_cast<const half_t *>(workspace), p.y, M, N / 2, s, /*interleaved=*/true);
        break;
    }
    default:
        return VQGEMM_E_VARIANT;
    }
    return static_cast<int>(e);
}

int vqgemm_e2e_gemm_b(const void *x, const void *codes, const void *codebook, void *y, int64_t M, int64_t K,
                      int64_t N, int32_t vec, int32_t entries, int32_t n_codebooks, int32_t code_bits,
                      int32_t variant, void *workspace, void *stream)
{
    return vqgemm_e2e_gemm_b_bias(x, codes, codebook, nullptr, y, M, K, N, vec, entries, n_codebooks, code_bits, variant,
                                  workspace, stream);
}

int vqgemm_e2e_gemm_a(const void *x, const void *w, const void *codebook, void *out, int64_t M, int64_t K,
                      int64_t Nc, int32_t variant, void *workspace, void *stream)
{
    if (M < 0 || K < 0 || Nc < 0 || M > INT_MAX / 2 || K > INT_MAX / 2 || Nc > INT_MAX / 4) return VQGEMM_E_SHAPE;
    if (Nc % 4 != 0) return VQGEMM_E_SHAPE;
    if (variant < VQGEMM_VARIANT_AUTO || variant > VQGEMM_VARIANT_TWOPASS) return VQGEMM_E_VARIANT;
    if (M == 0 || Nc == 0) return VQGEMM_OK;
    if (!out || !codebook || (K > 0 && (!x || !w))) return VQGEMM_E_NULL;
    if (!aligned(x, 2) || !aligned(out, 4) || !aligned(codebook, 4)) return VQGEMM_E_ALIGN;
    ProblemA p;
    p.x = static_cast<const half_t *>(x);
    p.w = static_cast<const uint8_t *>(w);
    p.cb = static_cast<const half_t *>(codebook);
    p.y = static_cast<half_t *>(out);
    p.M = (int)M; p.K = (int)K; p.Nc = (int)Nc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e = hipSuccess;
    // The fused tiled kernel where it applies and is expected to win; otherwise, with scratch, the
    // two-pass route (bit-exact dequant, then the MFMA GEMM), and without it the scalar kernel.
    if (variant == VQGEMM_VARIANT_AUTO) {
        if (fused_a_preferred(p, workspace != nullptr)) variant = VQGEMM_VARIANT_PREFILL;
        else variant = workspace ? VQGEMM_VARIANT_TWOPASS : VQGEMM_VARIANT_GENERIC;
    }
    switch (variant) {
    case VQGEMM_VARIANT_GENERIC:
        e = launch_generic_a(p, s);
        break;
    case VQGEMM_VARIANT_PREFILL:
        if (!fused_a_supports(p)) return aligned(x, 16) && aligned(w, 16) && aligned(codebook, 16) ? VQGEMM_E_VARIANT : VQGEMM_E_ALIGN;
        e = launch_fused_a(p, s);
        break;
    case VQGEMM_VARIANT_TWOPASS:
        if (!workspace) return VQGEMM_E_NULL;
        if (!aligned(workspace, 16)) return VQGEMM_E_ALIGN;
        e = launch_dequant_a(p, static_cast<half_t *>(workspace), s);
        if (e == hipSuccess)
            e = launch_gemm_nn(p.x, static_cast<const half_t *>(workspace), p.y, p.M, p.K, 2 * p.Nc, s);
        break;
    default:
        return VQGEMM_E_VARIANT;  // the decode tilings are geometry-B kernels
    }
    return static_cast<int>(e);
}

int vqgemm_select_variant_a(int64_t M, int64_t K, int64_t Nc, int32_t has_workspace)
{
    if (M < 0 || K < 0 || Nc < 0 || M > INT_MAX / 2 || K > INT_MAX / 2 || Nc > INT_MAX / 4 || Nc % 4 != 0) return VQGEMM_E_SHAPE;
    ProblemA p = {};
    p.M = (int)M; p.K = (int)K; p.Nc = (int)Nc;
    if (fused_a_preferred(p, has_workspace != 0)) return VQGEMM_VARIANT_PREFILL;
    return has_workspace ? VQGEMM_VARIANT_TWOPASS : VQGEMM_VARIANT_GENERIC;
}

int vqgemm_dequant_b(const void *codes, const void *codebook, void *w_out, int64_t N, int64_t K, int32_t vec,
                     int32_t entries, int32_t n_codebooks, int32_t code_bits, void *stream)
{
    const int rc = check_b(0, K, N, vec, entries, n_codebooks, code_bits);
    if (rc != VQGEMM_OK) return rc;
    if (N == 0 || K == 0) return VQGEMM_OK;
    if (!codes || !codebook || !w_out) return VQGEMM_E_NULL;
    if (!aligned(w_out, 2) || !aligned(codebook, 2) || !aligned(codes, code_bits / 8)) return VQGEMM_E_ALIGN;
    const ProblemB p = make_b(nullptr, codes, codebook, nullptr, 0, K, N, vec, entries, n_codebooks, code_bits);
    return static_cast<int>(launch_dequant_b(p, static_cast<half_t *>(w_out), static_cast<hipStream_t>(stream)));
}

int vqgemm_pack_codes_b(const void *codes, void *codes_out, int64_t N, int64_t K, int32_t vec, int32_t code_bits,
                        int32_t inverse, void *stream)
{
    if (N < 0 || K < 0 || N > INT_MAX / 2 || K > INT_MAX / 2) return VQGEMM_E_SHAPE;
    if (code_bits != 8 && code_bits != 16) return VQGEMM_E_CODEBITS;
    if (vec < 1 || K % vec != 0) return VQGEMM_E_SHAPE;
    if (!pack_codes_supports(N, K, vec, code_bits)) return VQGEMM_E_VARIANT;
    if (N == 0 || K == 0) return VQGEMM_OK;
    if (!codes || !codes_out) return VQGEMM_E_NULL;
    if (codes == codes_out) return VQGEMM_E_NULL;  // not in place: a permutation of the whole matrix
    if (!aligned(codes, 16) || !aligned(codes_out, 16)) return VQGEMM_E_ALIGN;
    return static_cast<int>(launch_pack_codes(codes, codes_out, N, K, vec, code_bits, inverse != 0,
                                              static_cast<hipStream_t>(stream)));
}

int vqgemm_decode_packed_supports(int64_t M, int64_t K, int64_t N, int32_t vec, int32_t entries, int32_t n_codebooks,
                                  int32_t code_bits)
{
    const int rc = check_b(M, K, N, vec, entries, n_codebooks, code_bits);
    if (rc != VQGEMM_OK) return rc;
    if (M == 0 || N == 0 || K == 0) return 0;
    ProblemB p = make_b(nullptr, nullptr, nullptr, nullptr, M, K, N, vec, entries, n_codebooks, code_bits);
    p.packed = true;
    return decode_packed_supports(p) ? 1 : 0;
}

int vqgemm_encode_b(const void *w, const void *codebook, void *codes_out, int64_t N, int64_t K, int32_t vec,
                    int32_t entries, int32_t n_codebooks, int32_t code_bits, void *stream)
{
    const int rc = check_b(0, K, N, vec, entries, n_codebooks, code_bits);
    if (rc != VQGEMM_OK) return rc;
    if (N == 0 || K == 0) return VQGEMM_OK;
    if (!w || !codebook || !codes_out) return VQGEMM_E_NULL;
    if (!aligned(w, 2) || !aligned(codebook, 2) || !aligned(codes_out, code_bits / 8)) return VQGEMM_E_ALIGN;
    const ProblemB p = make_b(nullptr, nullptr, codebook, nullptr, 0, K, N, vec, entries, n_codebooks, code_bits);
    if (!encode_supports(p)) return VQGEMM_E_VARIANT;
    return static_cast<int>(launch_encode_b(static_cast<const half_t *>(w), p, codes_out, static_cast<hipStream_t>(stream)));
}

int vqgemm_silu_mul(const void *gate_up, void *out, int64_t M, int64_t N, void *stream)
{
    if (M < 0 || N < 0 || M > INT_MAX / 2 || N > INT_MAX / 4) return VQGEMM_E_SHAPE;
    if (M == 0 || N == 0) return VQGEMM_OK;
    if (!gate_up || !out) return VQGEMM_E_NULL;
    if (!aligned(gate_up, 2) || !aligned(out, 2)) return VQGEMM_E_ALIGN;
    return static_cast<int>(launch_silu_mul(static_cast<const half_t *>(gate_up), static_cast<half_t *>(out), M, N,
                                            static_cast<hipStream_t>(stream)));
}

int vqgemm_max_code(const void *codes, int64_t count, int32_t code_bits, void *max_out, void *stream)
{
    if (count < 0) return VQGEMM_E_SHAPE;
    if (code_bits != 8 && code_bits != 16) return VQGEMM_E_CODEBITS;
    if (!max_out || (count > 0 && !codes)) return VQGEMM_E_NULL;
    if (!aligned(max_out, 4) || !aligned(codes, code_bits / 8)) return VQGEMM_E_ALIGN;
    return static_cast<int>(launch_max_code(codes, count, code_bits, static_cast<uint32_t *>(max_out),
                                            static_cast<hipStream_t>(stream)));
}

int vqgemm_dequant_a(const void *w, const void *codebook, void *w_out, int64_t K, int64_t Nc, void *stream)
{
    if (K < 0 || Nc < 0 || K > INT_MAX / 2 || Nc > INT_MAX / 4 || Nc % 4 != 0) return VQGEMM_E_SHAPE;
    if (K == 0 || Nc == 0) return VQGEMM_OK;
    if (!w || !codebook || !w_out) return VQGEMM_E_NULL;
    if (!aligned(w_out, 4) || !aligned(codebook, 4)) return VQGEMM_E_ALIGN;
    ProblemA p;
    p.x = nullptr;
    p.w = static_cast<const uint8_t *>(w);
    p.cb = static_cast<const half_t *>(codebook);
    p.y = nullptr;
    p.M = 0; p.K = (int)K; p.Nc = (int)Nc;
    return static_cast<int>(launch_dequant_a(p, static_cast<half_t *>(w_out), static_cast<hipStream_t>(stream)));
}

int vqgemm_gemm_f16(const void *x, const void *w, void *y, int64_t M, int64_t K, int64_t N, void *stream)
{
    if (M < 0 || K < 0 || N < 0 || M > INT_MAX / 2 || K > INT_MAX / 2 || N > INT_MAX / 2) return VQGEMM_E_SHAPE;
    if (M == 0 || N == 0) return VQGEMM_OK;
    if (!y || (K > 0 && (!x || !w))) return VQGEMM_E_NULL;
    if (!aligned(x, 2) || !aligned(w, 2) || !aligned(y, 2)) return VQGEMM_E_ALIGN;
    return static_cast<int>(launch_gemm_nn(static_cast<const half_t *>(x), static_cast<const half_t *>(w),
                                           static_cast<half_t *>(y), (int)M, (int)K, (int)N,
                                           static_cast<hipStream_t>(stream)));
}

}  // extern "C"
