// Concat, Slice and element-wise scalar nodes (host side).
// Contracts: reference src/dR_nodes_transform.c:8-232 (Slice), :238-569 (Concat),
// src/dR_nodes_math.c:259-527 (ElemWise1Op), src/dR_nodes_misc.c:1046-1546 (Normalization).
#include "dr_internal.hpp"

using namespace dr;

namespace {

gboolean nothing(dR_Graph*, dR_Node*) { return TRUE; }
gint32 out_volume(dR_Node* n) { return n->oshape.s0 * n->oshape.s1 * n->oshape.s2; }
gboolean free_layer(dR_Graph*, dR_Node* node) { free(node->layer); node->layer = NULL; return TRUE; }
inline int dim_of(const dR_Shape3& s, int d) { return d == 0 ? s.s0 : d == 1 ? s.s1 : s.s2; }

// ================================ Concat =========================================================

inline dR_Concat_Data* concat_of(dR_Node* n) { return (dR_Concat_Data*)n->layer; }

gboolean concat_propagate(dR_Graph* net, dR_Node* node) {
    dR_Concat_Data* c = concat_of(node);
    if (c->concatDim < 0 || c->concatDim > 2) { say("Concat Layer Error: concat dimension %d out of range!\n", c->concatDim); return FALSE; }
    std::vector<dR_Node*> ins = nodes_of(node->previous_layers);
    if ((int)ins.size() != c->n) {
        if (verbose(net)) say("Concat Layer Error: Parameter n does not match number of given inputnodes!\n");
        return FALSE;
    }
    node->oshape = ins[0]->oshape;
    int total = 0;
    for (dR_Node* in : ins) {
        for (int d = 0; d < 3; ++d)
            if (d != c->concatDim && dim_of(in->oshape, d) != dim_of(ins[0]->oshape, d)) {
                say("Concat Layer %d: inputs differ in dimension %d (%d vs %d)!\n", node->layerID, d,
                    dim_of(in->oshape, d), dim_of(ins[0]->oshape, d));
                return FALSE;
            }
        total += dim_of(in->oshape, c->concatDim);
    }
    ((gint*)&node->oshape)[c->concatDim] = total;
    return TRUE;
}

gboolean concat_schedule(dR_Graph* net, dR_Node* node) {
    dR_Concat_Data* c = concat_of(node);
    free(c->inputSizesInConcatDim);
    c->inputSizesInConcatDim = (gint*)malloc(sizeof(gint) * (size_t)c->n);
    c->maxInputSizeInConcatDim = 0;
    int i = 0;
    for (dR_Node* in : nodes_of(node->previous_layers)) {
        c->inputSizesInConcatDim[i] = dim_of(in->oshape, c->concatDim);
        if (c->inputSizesInConcatDim[i] > c->maxInputSizeInConcatDim) c->maxInputSizeInConcatDim = c->inputSizesInConcatDim[i];
        ++i;
    }
    if (debug(net)) say("Concat maxInputSizeInConcatDim: %d \n", c->maxInputSizeInConcatDim);
    return TRUE;
}

gboolean concat_compute(dR_Graph* net, dR_Node* node) {
    dR_Concat_Data* c = concat_of(node);
    if (c->drFused) return TRUE;       // the producers already wrote into this node's buffer
    int off[3] = { 0, 0, 0 };
    for (dR_Node* in : nodes_of(node->previous_layers)) {
        int rc = drhip_copy3d_f32(dev_out(in), in->oshape.s0, in->oshape.s1, 0, 0, 0,
                                  dev_out(node), node->oshape.s0, node->oshape.s1, off[0], off[1], off[2],
                                  in->oshape.s0, in->oshape.s1, in->oshape.s2, stream_of(net));
        if (device_failed(net, rc, "deepRACIN:concat")) return FALSE;
        off[c->concatDim] += dim_of(in->oshape, c->concatDim);
    }
    return TRUE;
}

gboolean concat_cleanup_layer(dR_Graph*, dR_Node* node) {
    free(concat_of(node)->inputSizesInConcatDim);
    free(node->layer);
    node->layer = NULL;
    return TRUE;
}

gchar* concat_serialize(dR_Node* node, gchar* params[], gint* numParams, gfloat*[], gint[], gint* numVariables) {
    dR_Concat_Data* c = concat_of(node);
    if (*numParams < 2) { say("SerializeNode needs space for 2 parameters and 0 variables!\n"); return NULL; }
    params[0] = fmt_dup("%d", c->n);
    params[1] = fmt_dup("%d", c->concatDim);
    *numParams = 2;
    *numVariables = 0;
    return (gchar*)"Concat";
}

gchar* concat_print(dR_Node* node) {
    dR_Concat_Data* c = concat_of(node);
    return fmt_dup("Concat Layer: %d\n Concat Dimension: %d\n Number of concatenated slices: %d\n", node->layerID, c->concatDim, c->n);
}

// ================================ Slice ==========================================================

inline dR_Slice_Data* slice_of(dR_Node* n) { return (dR_Slice_Data*)n->layer; }

gboolean slice_propagate(dR_Graph* net, dR_Node* node) {
    dR_Slice_Data* s = slice_of(node);
    if (node->previous_layers->length != 1 && verbose(net))
        say("Extract Slice Node with id %d has %d inputs but needs 1!\n", node->layerID, node->previous_layers->length);
    dR_Node* in = first_input(node);
    if (!in) return FALSE;
    s->ishape.s0 = in->oshape.s0; s->ishape.s1 = in->oshape.s1; s->ishape.s2 = in->oshape.s2; s->ishape.s3 = 0;
    node->oshape.s0 = s->oshape.s0; node->oshape.s1 = s->oshape.s1; node->oshape.s2 = s->oshape.s2;
    const bool inside = s->origin.s0 >= 0 && s->origin.s1 >= 0 && s->origin.s2 >= 0 &&
                        s->oshape.s0 > 0 && s->oshape.s1 > 0 && s->oshape.s2 > 0 &&
                        s->origin.s0 + s->oshape.s0 <= s->ishape.s0 && s->origin.s1 + s->oshape.s1 <= s->ishape.s1 &&
                        s->origin.s2 + s->oshape.s2 <= s->ishape.s2;
    if (!inside) { say("Slice Node %d: box leaves its input! \n", node->layerID); return FALSE; }
    return TRUE;
}

gboolean slice_compute(dR_Graph* net, dR_Node* node) {
    dR_Slice_Data* s = slice_of(node);
    int rc = drhip_copy3d_f32(dev_out(first_input(node)), s->ishape.s0, s->ishape.s1, s->origin.s0, s->origin.s1, s->origin.s2,
                              dev_out(node), s->oshape.s0, s->oshape.s1, 0, 0, 0,
                              s->oshape.s0, s->oshape.s1, s->oshape.s2, stream_of(net));
    return !device_failed(net, rc, "deepRACIN:extractSlice");
}

gchar* slice_serialize(dR_Node* node, gchar* params[], gint* numParams, gfloat*[], gint[], gint* numVariables) {
    dR_Slice_Data* s = slice_of(node);
    if (*numParams < 8) { say("SerializeNode needs space for 8 parameters and 0 variables!\n"); return NULL; }
    const int vals[8] = { s->origin.s0, s->origin.s1, s->origin.s2, s->origin.s3, s->oshape.s0, s->oshape.s1, s->oshape.s2, s->oshape.s3 };
    for (int i = 0; i < 8; ++i) params[i] = fmt_dup("%d", vals[i]);
    *numParams = 8;
    *numVariables = 0;
    return (gchar*)"Slice";
}

gchar* slice_print(dR_Node* node) {
    dR_Slice_Data* s = slice_of(node);
    return fmt_dup("Extract Slice Node: %d\n Origin: [%d, %d, %d, %d]\n Size: [%d, %d, %d, %d]\n", node->layerID,
                   s->origin.s0, s->origin.s1, s->origin.s2, s->origin.s3, s->oshape.s0, s->oshape.s1, s->oshape.s2, s->oshape.s3);
}

// ================================ ElemWise1Op ====================================================

inline dR_ElemWise1Op_Data* ew_of(dR_Node* n) { return (dR_ElemWise1Op_Data*)n->layer; }

gboolean ew_propagate(dR_Graph* net, dR_Node* node) {
    dR_ElemWise1Op_Data* e = ew_of(node);
    if (node->previous_layers->length != 1 && verbose(net))
        say("ElemWise1Op Node with id %d has %d inputs but needs 1!\n", node->layerID, node->previous_layers->length);
    dR_Node* in = first_input(node);
    if (!in) return FALSE;
    e->ishape = in->oshape;
    node->oshape = in->oshape;
    return TRUE;
}

gboolean ew_compute(dR_Graph* net, dR_Node* node) {
    dR_ElemWise1Op_Data* e = ew_of(node);
    int rc = drhip_scalar_op_f32(dev_out(first_input(node)), dev_out(node), (size_t)out_volume(node), (int)e->op, e->scalar, stream_of(net));
    return !device_failed(net, rc, "deepRACIN:elemwise1op");
}

gchar* ew_serialize(dR_Node* node, gchar* params[], gint* numParams, gfloat*[], gint[], gint* numVariables) {
    dR_ElemWise1Op_Data* e = ew_of(node);
    if (*numParams < 2) { say("SerializeNode needs space for 2 parameters and 0 variables!\n"); return NULL; }
    params[0] = fmt_dup("%d", (int)e->op);
    params[1] = fmt_dup("%f", e->scalar);
    *numParams = 2;
    *numVariables = 0;
    return (gchar*)"ElemWise1Op";
}

gchar* ew_print(dR_Node* node) {
    dR_ElemWise1Op_Data* e = ew_of(node);
    static const char* ops[] = { "AddS", "SubS", "MulS", "DivS", "Log", "Exp", "Sqrt", "Fill", "PowS" };
    return fmt_dup("Element-wise 1-operation node: %d\n Operation: %s\n Scalar: %f\n", node->layerID, ops[(unsigned)e->op % 9], e->scalar);
}

// ================================ Normalization ==================================================

inline dR_Normalization_Data* norm_of(dR_Node* n) { return (dR_Normalization_Data*)n->layer; }

gboolean norm_propagate(dR_Graph* net, dR_Node* node) {
    if (node->previous_layers->length != 1 && verbose(net))
        say("Normalization Layer with id %d has %d inputs but needs 1!\n", node->layerID, node->previous_layers->length);
    dR_Node* in = first_input(node);
    if (!in) return FALSE;
    norm_of(node)->ishape = in->oshape;
    node->oshape = in->oshape;
    return TRUE;
}

gboolean norm_allocate(dR_Graph* net, dR_Node* node) {
    dR_Normalization_Data* d = norm_of(node);
    return dR_createFloatBuffer(net, &d->tempFloatBuffer1, (gint)drhip_normalize_scratch_floats((size_t)out_volume(node)), CL_MEM_READ_WRITE);
}

gboolean norm_compute(dR_Graph* net, dR_Node* node) {
    dR_Normalization_Data* d = norm_of(node);
    int rc = drhip_normalize_f32(dev_out(first_input(node)), dev_out(node), (size_t)out_volume(node), (int)d->type,
                                 d->targetMean, d->targetDev, (float*)d->tempFloatBuffer1, stream_of(net));
    return !device_failed(net, rc, "deepRACIN:normalization");
}

gboolean norm_cleanup_buffers(dR_Graph* net, dR_Node* node) {
    dR_Normalization_Data* d = norm_of(node);
    gboolean ok = dR_clMemoryBufferCleanup(net, d->tempFloatBuffer1);
    d->tempFloatBuffer1 = NULL;
    return ok;
}

gchar* norm_serialize(dR_Node* node, gchar* params[], gint* numParams, gfloat*[], gint[], gint* numVariables) {
    dR_Normalization_Data* d = norm_of(node);
    if (*numParams < 3) { say("SerializeNode needs space for 3 parameters and 0 variables!\n"); return NULL; }
    params[0] = fmt_dup("%d", (int)d->type);
    params[1] = fmt_dup("%f", d->targetMean);
    params[2] = fmt_dup("%f", d->targetDev);
    *numParams = 3;
    *numVariables = 0;
    return (gchar*)"Normalization";
}

gchar* norm_print(dR_Node* node) {
    dR_Normalization_Data* d = norm_of(node);
    static const char* kinds[] = { "Mean", "Deviation", "Mean and deviation" };
    return fmt_dup("Normalization Layer: %d\n Type: %s\n Target mean: %f\n Target deviation: %f\n", node->layerID,
                   kinds[(unsigned)d->type % 3], d->targetMean, d->targetDev);
}

}  // namespace

extern "C" {

dR_Node* dR_Normalization(dR_Graph* net, dR_Node* inputLayer, dR_NormalizationType type, gfloat targetMean, gfloat targetDev) {
    dR_Normalization_Data* d = zalloc<dR_Normalization_Data>();
    dR_Node* n = zalloc<dR_Node>();
    d->type = type;
    d->targetMean = targetMean;
    d->targetDev = targetDev;
    n->layer = d;
    n->type = tNormalization;
    n->compute = norm_compute;
    n->schedule = nothing;
    n->propagateShape = norm_propagate;
    n->getRequiredOutputBufferSize = out_volume;
    n->createKernel = nothing;
    n->allocateBuffers = norm_allocate;
    n->fillBuffers = nothing;
    n->cleanupBuffers = norm_cleanup_buffers;
    n->cleanupLayer = free_layer;
    n->serializeNode = norm_serialize;
    n->parseAppendNode = dR_norm_parseAppendNode;
    n->printLayer = norm_print;
    link_single_input(n, inputLayer, "Normalization Layer");
    dR_appendLayer(net, n);
    return n;
}

dR_Node* dR_norm_parseAppendNode(dR_Graph* net, dR_Node** iNodes, gint numINodes, gchar** params, gint numParams,
                                 gfloat**, gint numVariables) {
    if (numINodes != 1) { say("Parsing Error: Normalization Node needs 1 InputNodes but got %d!\n", numINodes); return NULL; }
    if (numParams != 3 || numVariables != 0) { say("Parsing Error: Normalization Node needs 3 Parameters and 0 Variables!\n"); return NULL; }
    const int type = atoi(params[0]);
    if (type < 0 || type > 2) { say("Parsing Error: Normalization type %d unknown!\n", type); return NULL; }
    return dR_Normalization(net, iNodes[0], (dR_NormalizationType)type, (gfloat)atof(params[1]), (gfloat)atof(params[2]));
}

dR_Node* dR_Concat(dR_Graph* net, dR_Node** inputNodes, gint n, gint concatDim) {
    dR_Concat_Data* c = zalloc<dR_Concat_Data>();
    dR_Node* node = zalloc<dR_Node>();
    c->n = n;
    c->concatDim = concatDim;
    node->layer = c;
    node->type = tConcat;
    node->compute = concat_compute;
    node->schedule = concat_schedule;
    node->propagateShape = concat_propagate;
    node->getRequiredOutputBufferSize = out_volume;
    node->createKernel = nothing;
    node->allocateBuffers = nothing;
    node->fillBuffers = nothing;
    node->cleanupBuffers = nothing;
    node->cleanupLayer = concat_cleanup_layer;
    node->serializeNode = concat_serialize;
    node->parseAppendNode = dR_concat_parseAppendNode;
    node->printLayer = concat_print;
    node->next_layers = dR_list_createEmptyList();
    node->previous_layers = dR_list_createEmptyList();
    // the reference accepts up to three inputs (src/dR_nodes_transform.c:266)
    if (inputNodes != NULL && n > 0 && n < 4 && inputNodes[n - 1] != NULL) {
        for (int i = 0; i < n; ++i) {
            dR_list_append(node->previous_layers, inputNodes[i]);
            dR_list_append(inputNodes[i]->next_layers, node);
        }
    } else {
        say("Error: Concat node layer needs an appropriate number (n) of Inputnodes and n has to be 0<=n<4 \n");
    }
    dR_appendLayer(net, node);
    return node;
}

dR_Node* dR_concat_parseAppendNode(dR_Graph* net, dR_Node** iNodes, gint numINodes, gchar** params, gint numParams,
                                   gfloat**, gint numVariables) {
    if (numParams != 2 || numVariables != 0) { say("Parsing Error: Concat Node needs 2 Parameters and 0 Variables!\n"); return NULL; }
    const int n = atoi(params[0]);
    if (numINodes != n) { say("Parsing Error: Concat Node needs %d InputNodes but got %d!\n", n, numINodes); return NULL; }
    return dR_Concat(net, iNodes, n, atoi(params[1]));
}

dR_Node* dR_Slice(dR_Graph* net, dR_Node* inputLayer, dR_Shape4* origin, dR_Shape4* shape) {
    dR_Slice_Data* s = zalloc<dR_Slice_Data>();
    dR_Node* n = zalloc<dR_Node>();
    s->origin = *origin;
    s->oshape = *shape;
    n->layer = s;
    n->type = tSlice;
    n->compute = slice_compute;
    n->schedule = nothing;
    n->propagateShape = slice_propagate;
    n->getRequiredOutputBufferSize = out_volume;
    n->createKernel = nothing;
    n->allocateBuffers = nothing;
    n->fillBuffers = nothing;
    n->cleanupBuffers = nothing;
    n->cleanupLayer = free_layer;
    n->serializeNode = slice_serialize;
    n->parseAppendNode = dR_slice_parseAppendNode;
    n->printLayer = slice_print;
    link_single_input(n, inputLayer, "Slice Node");
    dR_appendLayer(net, n);
    return n;
}

dR_Node* dR_slice_parseAppendNode(dR_Graph* net, dR_Node** iNodes, gint numINodes, gchar** params, gint numParams,
                                  gfloat**, gint numVariables) {
    if (numINodes != 1) { say("Parsing Error: Slice Node needs 1 InputNodes but got %d!\n", numINodes); return NULL; }
    if (numParams != 8 || numVariables != 0) { say("Parsing Error: Slice Node needs 8 Parameters and 0 Variables!\n"); return NULL; }
    dR_Shape4 origin = { atoi(params[0]), atoi(params[1]), atoi(params[2]), atoi(params[3]) };
    dR_Shape4 shape = { atoi(params[4]), atoi(params[5]), atoi(params[6]), atoi(params[7]) };
    return dR_Slice(net, iNodes[0], &origin, &shape);
}

dR_Node* dR_ElemWise1Operation(dR_Graph* net, dR_Node* inputLayer, dR_ElemWise1OperationType op, gfloat scalar) {
    dR_ElemWise1Op_Data* e = zalloc<dR_ElemWise1Op_Data>();
    dR_Node* n = zalloc<dR_Node>();
    e->op = op;
    e->scalar = scalar;
    n->layer = e;
    n->type = tElemWise1Op;
    n->compute = ew_compute;
    n->schedule = nothing;
    n->propagateShape = ew_propagate;
    n->getRequiredOutputBufferSize = out_volume;
    n->createKernel = nothing;
    n->allocateBuffers = nothing;
    n->fillBuffers = nothing;
    n->cleanupBuffers = nothing;
    n->cleanupLayer = free_layer;
    n->serializeNode = ew_serialize;
    n->parseAppendNode = dR_elemwise1op_parseAppendNode;
    n->printLayer = ew_print;
    link_single_input(n, inputLayer, "ElemWise1Operation node");
    dR_appendLayer(net, n);
    return n;
}

dR_Node* dR_elemwise1op_parseAppendNode(dR_Graph* net, dR_Node** iNodes, gint numINodes, gchar** params, gint numParams,
                                        gfloat**, gint numVariables) {
    if (numINodes != 1) { say("Parsing Error: ElemWise1Op Node needs 1 InputNodes but got %d!\n", numINodes); return NULL; }
    if (numParams != 2 || numVariables != 0) { say("Parsing Error: ElemWise1Op Node needs 2 Parameters and 0 Variables!\n"); return NULL; }
    const int op = atoi(params[0]);
    if (op < 0 || op > 8) { say("Parsing Error: ElemWise1Op operation %d unknown!\n", op); return NULL; }
    return dR_ElemWise1Operation(net, iNodes[0], (dR_ElemWise1OperationType)op, (gfloat)atof(params[1]));
}

// ---- node types outside the CNN layer path -----------------------------------------------------------
// The reference's ctypes wrapper resolves these names while it is imported
// (python/deepracin/__init__.py.in:146-211); they keep the reference's signatures, append nothing and
// return NULL, the way every constructor here reports a refused node.

static dR_Node* outside_layer_path(const char* what) {
    say("%s: node type outside the CNN layer path, not available in this build; no node appended.\n", what);
    return NULL;
}

dR_Node* dR_MaskDependentFilter(dR_Graph*, dR_Node*, dR_Node*, dR_Shape3*) { return outside_layer_path("dR_MaskDependentFilter"); }
void dR_MaskDependentFilter_setVariables(dR_Node*, gfloat*, gfloat*) { outside_layer_path("dR_MaskDependentFilter_setVariables"); }
dR_Node* dR_PerPixelFilter(dR_Graph*, dR_Node*, dR_Node*, dR_Shape4*, dR_Shape4*) { return outside_layer_path("dR_PerPixelFilter"); }
dR_Node* dR_ElemWise2Operation(dR_Graph*, dR_Node*, dR_Node*, dR_ElemWise2OperationType) { return outside_layer_path("dR_ElemWise2Operation"); }
dR_Node* dR_ResolveRoI(dR_Graph*, dR_Node*, dR_Shape3*) { return outside_layer_path("dR_ResolveRoI"); }
dR_Node* dR_RGB2gray(dR_Graph*, dR_Node*) { return outside_layer_path("dR_RGB2gray"); }
dR_Node* dR_Upscaling(dR_Graph*, dR_Node*, dR_UpscalingType, gint, gint) { return outside_layer_path("dR_Upscaling"); }
dR_Node* dR_LabelCreation(dR_Graph*, dR_Node*, dR_LabelCreationType, gfloat, gfloat, gfloat) { return outside_layer_path("dR_LabelCreation"); }
dR_Node* dR_CropOrPad(dR_Graph*, dR_Node*, dR_Shape3*) { return outside_layer_path("dR_CropOrPad"); }
// Called (not bound at import) by the wrapper's Conv2dTransposed(); unfinished in the reference itself.
dR_Node* dR_Conv2dTransposed(dR_Graph*, dR_Node*, dR_Shape4, dR_Shape4, dR_ActivationType, gboolean) { return outside_layer_path("dR_Conv2dTransposed"); }
void dR_Conv2dtransposed_setVariables(dR_Node*, gfloat*, gfloat*) { outside_layer_path("dR_Conv2dtransposed_setVariables"); }

}  // extern "C"
