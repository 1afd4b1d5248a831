// Calls between the translation units of librocmlir_amd.so that are not part
// of its C ABI (the library is built with hidden visibility, so none of this
// is exported).
#pragma once
#include <stddef.h>

// Launches the handle's kernel once on `stream` with `workspace` standing in
// for the workspace pointer that rockamdLaunch's caller list would end with.
// `pointers` holds the problem's own pointers only (one fewer than
// rockamdLaunch takes when the problem has a workspace, the same otherwise).
// Fails with hipErrorInvalidValue, and a message for rockamdGetLastError, when
// the problem's workspace is larger than `capacity` bytes.  Allocates nothing
// once the handle's code object is loaded on the current device, which the
// first launch of a handle on a device does.
int rock_launch_with_workspace(void *handle, void *const *pointers, int num_pointers, void *workspace,
                               size_t capacity, void *stream);
