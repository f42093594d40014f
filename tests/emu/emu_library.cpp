// TEST INFRASTRUCTURE: the one translation unit of libhomcomp_emu.so that is not the library's own
// source: the globals of the execution model, and its allocator for the buffers a caller hands to
// the library.  They must come from here for two reasons: workgroups are processes, so whatever a
// kernel writes has to lie in shared memory for the caller to see it, and every access a kernel
// makes is checked against the list of allocations.
#define EMU_DEFINE_GLOBALS
#include "hip/hip_runtime.h"

extern "C" {

// `bytes` of zeroed "device memory" whose last byte lies in front of an inaccessible page
// (`align`: the alignment the end is rounded up to, 1 for byte streams); NULL when there is none.
void *emu_alloc_buffer(size_t bytes, size_t align)
{
    void *p = emu_device_alloc_named(bytes, "caller", align ? align : 1);
    if (p) memset(p, 0, bytes);
    return p;
}

int emu_free_buffer(void *p) { return emu_device_free(p) ? 0 : 1; }

int emu_live_allocations(void) { return emu_n_allocs; }

// bytes of "device memory" in use (what a free-memory query would be taken from)
size_t emu_live_bytes(void)
{
    const emu_locked lock(&emu_alloc_lock);
    size_t total = 0;
    for (int i = 0; i < emu_n_allocs; ++i) total += emu_allocs[i].hi - emu_allocs[i].lo;
    return total;
}

// Graph capture for the harness: between begin and end every launch the library makes is recorded
// instead of run; a replay runs the recorded launches in order, with their recorded arguments,
// on whatever the buffers hold then.
void *emu_graph_begin_capture(void) { return emu_capture_begin(); }
void *emu_graph_end_capture(void) { return emu_capture_end(); }
int emu_graph_launch(void *graph) { return emu_graph_replay((emu_graph *)graph) ? 0 : 1; }
int emu_graph_launches(void *graph) { return (int)((emu_graph *)graph)->launches.size(); }
void emu_graph_destroy(void *graph) { delete (emu_graph *)graph; }

}  // extern "C"
