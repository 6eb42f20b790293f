// Error reporting, version and row schedules of libfgnn_hip.so (host code only).
#include <algorithm>
#include <cstdarg>
#include <cstring>
#include <vector>
#include "fgnn_common.h"

static thread_local char g_err[512] = "";

void fgnn_set_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

extern "C" const char *fgnn_last_error(void) { return g_err; }
extern "C" int fgnn_version(void) { return 100; }

extern "C" int fgnn_schedule_create(const int32_t *ptr_dev, int n_rows, int seg_len, void *stream, fgnn_schedule_t **out)
{
    FGNN_REQUIRE(ptr_dev && out, FGNN_ERR_NULL, "fgnn_schedule_create: NULL argument");
    FGNN_REQUIRE(n_rows >= 0, FGNN_ERR_SHAPE, "fgnn_schedule_create: n_rows=%d", n_rows);
    if (seg_len <= 0) seg_len = 2048;
    seg_len = (seg_len + 63) & ~63;
    hipStream_t st = (hipStream_t)stream;
    std::vector<int32_t> ptr((size_t)n_rows + 1);
    FGNN_HIP(hipMemcpyAsync(ptr.data(), ptr_dev, sizeof(int32_t) * ((size_t)n_rows + 1), hipMemcpyDeviceToHost, st));
    FGNN_HIP(hipStreamSynchronize(st));
    FGNN_REQUIRE(ptr[0] == 0, FGNN_ERR_SHAPE, "fgnn_schedule_create: ptr[0]=%d, expected 0", ptr[0]);
    for (int i = 0; i < n_rows; ++i)
        FGNN_REQUIRE(ptr[i + 1] >= ptr[i], FGNN_ERR_SHAPE, "fgnn_schedule_create: ptr decreases at row %d", i);

    std::vector<fgnn_item> items;
    std::vector<fgnn_split> splits;
    items.reserve((size_t)n_rows + 1024);
    int n_part = 0;
    // segments of long rows first (they are the largest items), then whole rows, longest first
    for (int i = 0; i < n_rows; ++i) {
        int deg = ptr[i + 1] - ptr[i];
        if (deg <= seg_len) continue;
        int nseg = (deg + seg_len - 1) / seg_len;
        int len = (((deg + nseg - 1) / nseg) + 63) & ~63;
        nseg = (deg + len - 1) / len;
        splits.push_back({i, n_part, nseg, 0});
        for (int g = 0; g < nseg; ++g) {
            int b = ptr[i] + g * len;
            int e = std::min(ptr[i + 1], b + len);
            items.push_back({i, b, e, n_part++});
        }
    }
    size_t first_whole = items.size();
    for (int i = 0; i < n_rows; ++i) {
        int deg = ptr[i + 1] - ptr[i];
        if (deg <= seg_len) items.push_back({i, ptr[i], ptr[i + 1], -1});
    }
    std::stable_sort(items.begin() + first_whole, items.end(),
                     [](const fgnn_item &a, const fgnn_item &b) { return (a.end - a.begin) > (b.end - b.begin); });

    fgnn_schedule *s = new fgnn_schedule();
    s->n_rows = n_rows;
    s->n_edges = n_rows ? ptr[n_rows] : 0;
    s->seg_len = seg_len;
    s->n_items = (int)items.size();
    s->n_partials = n_part;
    s->n_split = (int)splits.size();
    s->items_dev = nullptr;
    s->split_dev = nullptr;
    s->ptr_dev = ptr_dev;
    (void)hipGetDevice(&s->device);
    hipError_t err = hipSuccess;
    if (!items.empty()) {
        err = hipMalloc((void **)&s->items_dev, items.size() * sizeof(fgnn_item));
        if (err == hipSuccess) err = hipMemcpyAsync(s->items_dev, items.data(), items.size() * sizeof(fgnn_item), hipMemcpyHostToDevice, st);
    }
    if (err == hipSuccess && !splits.empty()) {
        err = hipMalloc((void **)&s->split_dev, splits.size() * sizeof(fgnn_split));
        if (err == hipSuccess) err = hipMemcpyAsync(s->split_dev, splits.data(), splits.size() * sizeof(fgnn_split), hipMemcpyHostToDevice, st);
    }
    if (err == hipSuccess) err = hipStreamSynchronize(st);   // the host vectors die at return
    if (err != hipSuccess) {
        fgnn_set_error("fgnn_schedule_create: %s", hipGetErrorString(err));
        fgnn_schedule_destroy(s);
        return (int)err;
    }
    *out = s;
    return 0;
}

extern "C" void fgnn_schedule_destroy(fgnn_schedule_t *s)
{
    if (!s) return;
    if (s->items_dev) (void)hipFree(s->items_dev);
    if (s->split_dev) (void)hipFree(s->split_dev);
    delete s;
}

extern "C" int fgnn_schedule_num_items(const fgnn_schedule_t *s) { return s ? s->n_items : 0; }
extern "C" int fgnn_schedule_num_partials(const fgnn_schedule_t *s) { return s ? s->n_partials : 0; }
extern "C" int64_t fgnn_schedule_num_edges(const fgnn_schedule_t *s) { return s ? s->n_edges : 0; }
