// Internal helpers shared by the host-side graph code.  Nothing here touches HIP directly: the
// host side reaches the device only through the C-ABI in include/dr_hip.h.
#pragma once

#include "deepRACIN.h"

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

namespace dr {

// printf to stdout, the reference's only error/log channel (g_print).
inline void say(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vfprintf(stdout, fmt, ap);
    va_end(ap);
    fflush(stdout);
}

// printf into a malloc'ed string (callers of printLayer / serializeNode params own the result).
inline char* fmt_dup(const char* fmt, ...) {
    va_list ap, ap2;
    va_start(ap, fmt);
    va_copy(ap2, ap);
    int n = vsnprintf(nullptr, 0, fmt, ap);
    va_end(ap);
    char* out = (char*)malloc((size_t)n + 1);
    vsnprintf(out, (size_t)n + 1, fmt, ap2);
    va_end(ap2);
    return out;
}

template <typename T> inline T* zalloc(size_t n = 1) { return (T*)calloc(n, sizeof(T)); }

inline bool verbose(const dR_Graph* net) { return net && net->config && !net->config->silent; }
inline bool debug(const dR_Graph* net)   { return verbose(net) && net->config->debugInfo; }

// Walk a dR_List without disturbing its embedded cursor.
template <typename F> inline void for_each(const dR_List* l, F f) {
    if (!l) return;
    for (dR_ListElement* e = l->first; e; e = e->next) f(e->element);
}
inline std::vector<dR_Node*> nodes_of(const dR_List* l) {
    std::vector<dR_Node*> v;
    for_each(l, [&](void* p) { v.push_back((dR_Node*)p); });
    return v;
}
inline dR_Node* first_input(const dR_Node* n) {
    return (n->previous_layers && n->previous_layers->first) ? (dR_Node*)n->previous_layers->first->element : nullptr;
}

// Device address of a node's output storage.
inline float* dev_out(const dR_Node* n) { return (float*)(*n->outputBuf->bufptr); }
inline void*  stream_of(const dR_Graph* net) { return net->clConfig->hipStream; }

// Wire a single-input node behind `input` (the pattern every constructor of the reference repeats).
void link_single_input(dR_Node* node, dR_Node* input, const char* what);
// Report a failed drhip_* call the way dR_openCLError does: message to stdout, FALSE to the caller.
gboolean device_failed(dR_Graph* net, int status, const char* what);
// Copy caller-owned floats.
float* dup_floats(const float* src, size_t n);
// While dR_parseGraph builds a node, the float counts of the variable files it read for that node
// (0 = unknown, e.g. when a factory is called by user code).  Factories use it to refuse a file
// shorter than the tensor it is supposed to hold instead of reading past its end.
extern thread_local size_t parse_var_floats[2];
bool parsed_var_has(int which, size_t need_floats, const char* what);

}  // namespace dr

// graph.dr node factories (one per node description), used by the parser.
extern "C" {
dR_Node* dR_datafeednode_parseAppendNode(dR_Graph*, dR_Node**, gint, gchar**, gint, gfloat**, gint);
dR_Node* dR_conv2d_parseAppendNode(dR_Graph*, dR_Node**, gint, gchar**, gint, gfloat**, gint);
dR_Node* dR_pooling_parseAppendNode(dR_Graph*, dR_Node**, gint, gchar**, gint, gfloat**, gint);
dR_Node* dR_fc_parseAppendNode(dR_Graph*, dR_Node**, gint, gchar**, gint, gfloat**, gint);
dR_Node* dR_softmax_parseAppendNode(dR_Graph*, dR_Node**, gint, gchar**, gint, gfloat**, gint);
dR_Node* dR_concat_parseAppendNode(dR_Graph*, dR_Node**, gint, gchar**, gint, gfloat**, gint);
dR_Node* dR_slice_parseAppendNode(dR_Graph*, dR_Node**, gint, gchar**, gint, gfloat**, gint);
dR_Node* dR_elemwise1op_parseAppendNode(dR_Graph*, dR_Node**, gint, gchar**, gint, gfloat**, gint);
dR_Node* dR_norm_parseAppendNode(dR_Graph*, dR_Node**, gint, gchar**, gint, gfloat**, gint);
}
