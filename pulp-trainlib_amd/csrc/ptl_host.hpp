// Host-side helpers shared by the entry-point translation units.
#pragma once
#include "ptl_common.hpp"

#include <vector>

namespace ptl {

const char *last_error();
int last_status();
void set_status(int s);
int init_device(int device);
int dw_noalloc_setup(int device);  // looks up the fixed partial-sum array of the current device

// Maps caller pointers to device pointers.  Device pointers pass through;
// host pointers get a device buffer from a pool kept between calls, filled
// before the kernels run (copy_in) and copied back by finish() (copy_out).
// finish() synchronises only when something was staged.
class Stager {
   public:
    // device_only: host pointers are rejected instead of staged (callers that may not allocate)
    explicit Stager(bool device_only = false) : device_only_(device_only) {}
    ~Stager();
    Stager(const Stager &) = delete;
    Stager &operator=(const Stager &) = delete;

    template <typename T>
    const T *in(const T *p, size_t n) {
        return static_cast<const T *>(map(p, n * sizeof(T), true, false));
    }
    template <typename T>
    T *out(T *p, size_t n) {
        return static_cast<T *>(map(p, n * sizeof(T), false, true));
    }
    template <typename T>
    T *inout(T *p, size_t n) {
        return static_cast<T *>(map(p, n * sizeof(T), true, true));
    }
    bool failed() const { return failed_; }
    bool rejected() const { return rejected_; }  // failed because of the arguments, not because of HIP
    int finish(int rc);
    // Gives the staging buffers back without copying anything out (the kernels they were mapped for did not run).
    void discard();

   private:
    struct Item {
        void *host;
        void *dev;
        size_t bytes;
        bool copy_out;
        bool copied_in;
    };
    void *map(const void *p, size_t bytes, bool copy_in, bool copy_out);
    std::vector<Item> items_;
    bool failed_ = false;
    bool finished_ = false;
    bool device_only_ = false;
    bool rejected_ = false;
};

}  // namespace ptl
