// Doubly linked list with one embedded cursor, plus the two tiny matmul helpers.
// Behaviour follows the reference's list (src/dR_core.c:504-665): node plug-ins and user code
// iterate with dR_list_resetIt / dR_list_next, so the cursor rules are part of the contract:
//   - next() on a reset list yields the first element; after the last element it yields NULL and
//     resets itself;
//   - removing the element under the cursor moves the cursor one step back (or resets it when the
//     head was removed), so that the following next() yields the removed element's successor;
//   - pop() takes the head and, if the cursor sat on it, advances the cursor.
#include "dr_internal.hpp"

extern "C" {

dR_List* dR_list_createEmptyList(void) { return dr::zalloc<dR_List>(); }

void dR_list_append(dR_List* list, void* elem) {
    dR_ListElement* e = dr::zalloc<dR_ListElement>();
    e->element = elem;
    e->previous = list->last;
    if (list->last) list->last->next = e; else list->first = e;
    list->last = e;
    list->length++;
}

gboolean dR_list_removeFirstOcc(dR_List* list, void* elem) {
    for (dR_ListElement* e = list->first; e; e = e->next) {
        if (e->element != elem) continue;
        if (list->iterator == e) list->iterator = e->previous;   // NULL when e is the head
        if (e->previous) e->previous->next = e->next; else list->first = e->next;
        if (e->next) e->next->previous = e->previous; else list->last = e->previous;
        free(e);
        list->length--;
        return TRUE;
    }
    return FALSE;
}

void* dR_list_pop(dR_List* list) {
    dR_ListElement* head = list->first;
    if (!head) return NULL;
    void* payload = head->element;
    if (list->iterator == head) list->iterator = head->next;
    list->first = head->next;
    if (list->first) list->first->previous = NULL; else list->last = NULL;
    free(head);
    list->length--;
    return payload;
}

void* dR_list_next(dR_List* list) {
    list->iterator = list->iterator ? list->iterator->next : list->first;
    return list->iterator ? list->iterator->element : NULL;
}

void dR_list_resetIt(dR_List* list) { list->iterator = NULL; }

void dR_list_cleanup(dR_List* list) {
    if (!list) return;
    for (dR_ListElement* e = list->first; e;) {
        dR_ListElement* nxt = e->next;
        free(e);
        e = nxt;
    }
    free(list);
}

// result[r1 x c2] = mat1[r1 x c1] * mat2[r2 x c2]
gboolean dR_matmul(gfloat* mat1, gint mat1rows, gint mat1cols, gfloat* mat2, gint mat2rows,
                   gint mat2cols, gfloat* result) {
    if (mat1cols != mat2rows) { dr::say("Matmul failed: Dimensions not matching!\n"); return FALSE; }
    for (int r = 0; r < mat1rows; ++r)
        for (int c = 0; c < mat2cols; ++c) {
            float acc = 0.0f;
            for (int k = 0; k < mat1cols; ++k) acc += mat1[r * mat1cols + k] * mat2[k * mat2cols + c];
            result[r * mat2cols + c] = acc;
        }
    return TRUE;
}

// result[r1 x r2] = mat1[r1 x c1] * mat2[r2 x c2]^T
gboolean dR_matmulT(gfloat* mat1, gint mat1rows, gint mat1cols, gfloat* mat2, gint mat2rows,
                    gint mat2cols, gfloat* result) {
    if (mat1cols != mat2cols) { dr::say("MatmulT failed: Dimensions not matching!\n"); return FALSE; }
    for (int r = 0; r < mat1rows; ++r)
        for (int c = 0; c < mat2rows; ++c) {
            float acc = 0.0f;
            for (int k = 0; k < mat1cols; ++k) acc += mat1[r * mat1cols + k] * mat2[c * mat2cols + k];
            result[r * mat2rows + c] = acc;
        }
    return TRUE;
}

}  // extern "C"

namespace dr {

void link_single_input(dR_Node* node, dR_Node* input, const char* what) {
    node->previous_layers = dR_list_createEmptyList();
    node->next_layers = dR_list_createEmptyList();
    if (!input) {
        say("Error: %s needs an appropriate Inputnode\n", what);
        return;
    }
    dR_list_append(node->previous_layers, input);
    dR_list_append(input->next_layers, node);
}

gboolean device_failed(dR_Graph* net, int status, const char* what) {
    if (status == DRHIP_OK) return FALSE;
    if (net && net->clConfig) net->clConfig->clError = status;
    say("deepRACIN device error in %s: %s\n", what, drhip_last_error());
    return TRUE;
}

thread_local size_t parse_var_floats[2] = {0, 0};

bool parsed_var_has(int which, size_t need, const char* what) {
    if (parse_var_floats[which] == 0 || parse_var_floats[which] >= need) return true;
    say("Parsing Error: %s needs %zu floats but its variable file holds %zu!\n", what, need, parse_var_floats[which]);
    return false;
}

float* dup_floats(const float* src, size_t n) {
    float* p = (float*)malloc(n * sizeof(float));
    if (p && src) memcpy(p, src, n * sizeof(float));
    return p;
}

}  // namespace dr
