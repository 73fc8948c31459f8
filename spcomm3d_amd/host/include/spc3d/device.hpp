// RAII C++ handles over the C ABI (include/spcomm3d_hip.h) for callers that keep
// operands resident on the device across calls.  Header-only; every member is
// one C-ABI call, errors become exceptions.
#pragma once

#include <cstdint>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <utility>
#include <vector>

#include "../../../../include/spcomm3d_hip.h"

namespace spc3d {

// SPC3D_ERR_BAD_INDEX mirrors the reference's std::out_of_range from .at().
inline void check(int status, const char *call)
{
    if (status == SPC3D_OK)
        return;
    const std::string msg = std::string(call) + ": " + spc3d_status_name(status) + ": " +
                            spc3d_last_error();
    if (status == SPC3D_ERR_BAD_INDEX)
        throw std::out_of_range(msg);
    throw std::runtime_error(msg);
}

template <typename T> constexpr int dtype_of()
{
    static_assert(std::is_same<T, float>::value || std::is_same<T, double>::value,
                  "float or double");
    return std::is_same<T, double>::value ? SPC3D_F64 : SPC3D_F32;
}

class Context {
  public:
    explicit Context(int device = 0) { check(spc3d_ctx_create(device, &h_), "spc3d_ctx_create"); }
    // With explicit options (host threads of the one-shot calls, auxiliary stream, host cache).
    Context(int device, const spc3d_ctx_opts &opts)
    {
        check(spc3d_ctx_create_ex(device, &opts, &h_), "spc3d_ctx_create_ex");
    }
    ~Context()
    {
        if (h_)
            spc3d_ctx_destroy(h_);
    }
    Context(const Context &) = delete;
    Context &operator=(const Context &) = delete;
    spc3d_ctx *get() const { return h_; }
    void sync() { check(spc3d_ctx_sync(h_), "spc3d_ctx_sync"); }
    void mark(int slot) { check(spc3d_timer_mark(h_, slot), "spc3d_timer_mark"); }
    float elapsed_ms(int start, int stop)
    {
        float ms = 0;
        check(spc3d_timer_elapsed_ms(h_, start, stop, &ms), "spc3d_timer_elapsed_ms");
        return ms;
    }

  private:
    spc3d_ctx *h_ = nullptr;
};

template <typename T> class Panel {
  public:
    Panel(Context &ctx, uint32_t m, uint32_t n) : m_(m), n_(n)
    {
        check(spc3d_panel_create(ctx.get(), dtype_of<T>(), m, n, &h_), "spc3d_panel_create");
    }
    // Over the caller's device memory (spc3d_panel_wrap): nothing is copied or freed.
    Panel(Context &ctx, uint32_t m, uint32_t n, T *device_memory) : m_(m), n_(n)
    {
        check(spc3d_panel_wrap(ctx.get(), dtype_of<T>(), m, n, device_memory, &h_),
              "spc3d_panel_wrap");
    }
    ~Panel()
    {
        if (h_)
            spc3d_panel_destroy(h_);
    }
    Panel(const Panel &) = delete;
    Panel &operator=(const Panel &) = delete;
    spc3d_panel *get() const { return h_; }
    uint32_t rows() const { return m_; }
    uint32_t cols() const { return n_; }
    void upload(const T *host) { check(spc3d_panel_upload(h_, host), "spc3d_panel_upload"); }
    void download(T *host) { check(spc3d_panel_download(h_, host), "spc3d_panel_download"); }
    void fill(double v) { check(spc3d_panel_fill(h_, v), "spc3d_panel_fill"); }
    void copy_from(const Panel &src) { check(spc3d_panel_copy(h_, src.h_), "spc3d_panel_copy"); }

  private:
    spc3d_panel *h_ = nullptr;
    uint32_t m_, n_;
};

template <typename T> class Vals {
  public:
    Vals(Context &ctx, uint64_t n) : n_(n)
    {
        check(spc3d_vals_create(ctx.get(), dtype_of<T>(), n, &h_), "spc3d_vals_create");
    }
    // Over the caller's device memory (spc3d_vals_wrap): nothing is copied or freed.
    Vals(Context &ctx, uint64_t n, T *device_memory) : n_(n)
    {
        check(spc3d_vals_wrap(ctx.get(), dtype_of<T>(), n, device_memory, &h_), "spc3d_vals_wrap");
    }
    ~Vals()
    {
        if (h_)
            spc3d_vals_destroy(h_);
    }
    Vals(const Vals &) = delete;
    Vals &operator=(const Vals &) = delete;
    spc3d_vals *get() const { return h_; }
    uint64_t size() const { return n_; }
    void *device_ptr() const
    {
        void *p = nullptr;
        check(spc3d_vals_device_ptr(h_, &p), "spc3d_vals_device_ptr");
        return p;
    }
    void upload(const T *host) { check(spc3d_vals_upload(h_, host), "spc3d_vals_upload"); }
    void download(T *host) { check(spc3d_vals_download(h_, host), "spc3d_vals_download"); }
    void fill(double v) { check(spc3d_vals_fill(h_, v), "spc3d_vals_fill"); }

  private:
    spc3d_vals *h_ = nullptr;
    uint64_t n_;
};

template <typename T> class Plan {
  public:
    // vv may be null (set_values later); opts may be null (library defaults).
    Plan(Context &ctx, uint32_t nrows, uint32_t ncols, uint64_t nnz, const uint32_t *ii,
         const uint32_t *jj, const T *vv, const spc3d_plan_opts *opts = nullptr)
    {
        check(opts ? spc3d_plan_create_ex(ctx.get(), dtype_of<T>(), nrows, ncols, nnz, ii, jj, vv,
                                          opts, &h_)
                   : spc3d_plan_create(ctx.get(), dtype_of<T>(), nrows, ncols, nnz, ii, jj, vv,
                                       &h_),
              "spc3d_plan_create");
    }
    // A pattern that already lives on the device: dev_ii, dev_jj are device pointers
    // to nnz uint32 each.  The plan has no values until set_values.
    struct FromDevice {};
    Plan(FromDevice, Context &ctx, uint32_t nrows, uint32_t ncols, uint64_t nnz,
         const void *dev_ii, const void *dev_jj, const spc3d_plan_opts *opts = nullptr)
    {
        check(spc3d_plan_create_from_device(ctx.get(), dtype_of<T>(), nrows, ncols, nnz, dev_ii,
                                            dev_jj, opts, &h_),
              "spc3d_plan_create_from_device");
    }
    ~Plan()
    {
        if (h_)
            spc3d_plan_destroy(h_);
    }
    Plan(const Plan &) = delete;
    Plan &operator=(const Plan &) = delete;
    spc3d_plan *get() const { return h_; }
    void set_values(const T *vv) { check(spc3d_plan_set_values(h_, vv), "spc3d_plan_set_values"); }
    void set_values(const Vals<T> &vv)
    {
        check(spc3d_plan_set_values_device(h_, vv.get()), "spc3d_plan_set_values_device");
    }
    spc3d_plan_info info() const
    {
        spc3d_plan_info i;
        check(spc3d_plan_get_info(h_, &i), "spc3d_plan_get_info");
        return i;
    }

  private:
    spc3d_plan *h_ = nullptr;
};

// Buffer slot i <-> dense row rows[i] of a panel with panel_rows rows: the device
// form of SparseComm::sendptr / recvptr (src/comm.hpp:41,49).
class RowMap {
  public:
    RowMap(Context &ctx, uint32_t panel_rows, uint64_t n, const uint32_t *rows) : n_(n)
    {
        check(spc3d_rowmap_create(ctx.get(), panel_rows, n, rows, &h_), "spc3d_rowmap_create");
    }
    ~RowMap()
    {
        if (h_)
            spc3d_rowmap_destroy(h_);
    }
    RowMap(const RowMap &) = delete;
    RowMap &operator=(const RowMap &) = delete;
    spc3d_rowmap *get() const { return h_; }
    uint64_t size() const { return n_; }

  private:
    spc3d_rowmap *h_ = nullptr;
    uint64_t n_;
};

// buf[i,:] = P[rows[i],:]  (SparseComm::copy_to_sendbuff, src/comm.hpp:90-103)
template <typename T>
void rows_pack(Context &ctx, const Panel<T> &P, const RowMap &map, Vals<T> &buf)
{
    check(spc3d_rows_pack(ctx.get(), P.get(), map.get(), buf.get()), "spc3d_rows_pack");
}

// P[rows[i],:] = buf[i,:]  (SparseComm::copy_from_recvbuff, src/comm.hpp:166-177)
template <typename T>
void rows_unpack(Context &ctx, Panel<T> &P, const RowMap &map, const Vals<T> &buf)
{
    check(spc3d_rows_unpack(ctx.get(), P.get(), map.get(), buf.get()), "spc3d_rows_unpack");
}

// P[rows[i],:] += buf[i,:] in slot order  (SparseComm::SUM_from_recvbuff, src/comm.hpp:178-189)
template <typename T>
void rows_unpack_sum(Context &ctx, Panel<T> &P, const RowMap &map, const Vals<T> &buf)
{
    check(spc3d_rows_unpack_sum(ctx.get(), P.get(), map.get(), buf.get()),
          "spc3d_rows_unpack_sum");
}

// C = S .* (A B^T) on resident operands; asynchronous on the context's stream.
template <typename T>
void sddmm(Context &ctx, Plan<T> &S, const Panel<T> &A, const Panel<T> &B, Vals<T> &C)
{
    check(spc3d_sddmm(ctx.get(), S.get(), A.get(), B.get(), C.get()), "spc3d_sddmm");
}

// Y += A X on resident operands; asynchronous on the context's stream.
template <typename T> void spmm(Context &ctx, Plan<T> &A, const Panel<T> &X, Panel<T> &Y)
{
    check(spc3d_spmm(ctx.get(), A.get(), X.get(), Y.get()), "spc3d_spmm");
}

// Both of the above over one pattern and one B in a single pass (spc3d_sddmm_spmm):
// C as sddmm; Y += S B, or Y += C B when chained.
template <typename T>
void sddmm_spmm(Context &ctx, Plan<T> &S, const Panel<T> &A, const Panel<T> &B, Vals<T> &C,
                Panel<T> &Y, bool chained = false)
{
    check(spc3d_sddmm_spmm(ctx.get(), S.get(), A.get(), B.get(), C.get(), Y.get(), chained ? 1 : 0),
          "spc3d_sddmm_spmm");
}

} // namespace spc3d
