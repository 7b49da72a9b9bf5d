// Pooling, FullyConnected and Softmax nodes (host side).
// Contracts: reference src/dR_nodes_pooling.c:5-224, src/dR_nodes_fc.c:6-306, src/dR_nodes_math.c:529-767.
#include "dr_internal.hpp"

using namespace dr;

namespace {

gboolean nothing(dR_Graph*, dR_Node*) { return TRUE; }
gint32 out_volume(dR_Node* n) { return n->oshape.s0 * n->oshape.s1 * n->oshape.s2; }
inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// ================================ Pooling ========================================================

inline dR_Pooling_Data* pool_of(dR_Node* n) { return (dR_Pooling_Data*)n->layer; }

gboolean pool_propagate(dR_Graph* net, dR_Node* node) {
    dR_Pooling_Data* p = pool_of(node);
    if (node->previous_layers->length != 1 && verbose(net))
        say("Pooling Layer with id %d has %d inputs but needs 1!\n", node->layerID, node->previous_layers->length);
    dR_Node* in = first_input(node);
    if (!in) return FALSE;
    p->ishape = in->oshape;
    if (p->stride.s1 <= 0 || p->stride.s2 <= 0 || p->stride.s3 <= 0 || p->shape.s1 <= 0 || p->shape.s2 <= 0 || p->shape.s3 <= 0) {
        if (verbose(net)) say("Pooling window and stride must be positive! \n");
        return FALSE;
    }
    node->oshape.s0 = ceil_div(p->ishape.s0, p->stride.s1);
    node->oshape.s1 = ceil_div(p->ishape.s1, p->stride.s2);
    node->oshape.s2 = ceil_div(p->ishape.s2, p->stride.s3);
    if (node->oshape.s0 <= 0 || node->oshape.s1 <= 0 || node->oshape.s2 <= 0) {
        if (verbose(net)) say("Pooling Shape propagates to Zero. False shape parameters! \n");
        return FALSE;
    }
    return TRUE;
}

gboolean pool_schedule(dR_Graph* net, dR_Node* node) {
    dR_Pooling_Data* p = pool_of(node);
    p->useLMEM = FALSE;
    if (p->poolingType != tMax && p->poolingType != tAverage) {
        say("Pooling Layer %d: pooling type %d is not implemented (0 max, 1 average)! \n", node->layerID, (int)p->poolingType);
        return FALSE;
    }
    if (debug(net)) say("Scheduled Pooling Layer \n");
    return TRUE;
}

gboolean pool_compute(dR_Graph* net, dR_Node* node) {
    dR_Pooling_Data* p = pool_of(node);
    if (p->drFused) return TRUE;        // the convolution in front stored the pooled tensor already
    int rc = drhip_pool_f32(dev_out(first_input(node)), dev_out(node), NULL, p->ishape.s0, p->ishape.s1, p->ishape.s2,
                            p->shape.s1, p->shape.s2, p->shape.s3, p->stride.s1, p->stride.s2, p->stride.s3,
                            (int)p->poolingType, stream_of(net));
    return !device_failed(net, rc, "deepRACIN:pool");
}

gchar* pool_serialize(dR_Node* node, gchar* params[], gint* numParams, gfloat*[], gint[], gint* numVariables) {
    dR_Pooling_Data* p = pool_of(node);
    if (*numParams < 9) { say("SerializeNode needs space for 9 parameters and 0 variables!\n"); return NULL; }
    const int vals[9] = { (int)p->poolingType, p->shape.s0, p->shape.s1, p->shape.s2, p->shape.s3,
                          p->stride.s0, p->stride.s1, p->stride.s2, p->stride.s3 };
    for (int i = 0; i < 9; ++i) params[i] = fmt_dup("%d", vals[i]);
    *numParams = 9;
    *numVariables = 0;
    return (gchar*)"Pooling";
}

gchar* pool_print(dR_Node* node) {
    dR_Pooling_Data* p = pool_of(node);
    const char* kind = p->poolingType == tMax ? "Max Pooling" : p->poolingType == tAverage ? "Average pooling" : "L2 norm pooling";
    return fmt_dup("Pooling Layer: %d\n Shape: %d, %d, %d, %d\n Pooling Type: %s\n Stride: %d, %d, %d, %d\n", node->layerID,
                   p->shape.s0, p->shape.s1, p->shape.s2, p->shape.s3, kind, p->stride.s0, p->stride.s1, p->stride.s2, p->stride.s3);
}

gboolean free_layer(dR_Graph*, dR_Node* node) { free(node->layer); node->layer = NULL; return TRUE; }

// ================================ FullyConnected =================================================

inline dR_FC_Data* fc_of(dR_Node* n) { return (dR_FC_Data*)n->layer; }

gboolean fc_propagate(dR_Graph* net, dR_Node* node) {
    dR_FC_Data* f = fc_of(node);
    if (node->previous_layers->length != 1 && verbose(net))
        say("FullyConnected Layer with id %d has %d inputs but needs 1!\n", node->layerID, node->previous_layers->length);
    dR_Node* in = first_input(node);
    if (!in) return FALSE;
    f->ishape = in->oshape;
    if (f->ishape.s0 * f->ishape.s1 * f->ishape.s2 != f->shape.s0) {
        if (verbose(net)) say("FullyConnected Layer does not match Input Size! \n");
        return FALSE;
    }
    if (f->shape.s1 <= 0) return FALSE;
    node->oshape.s0 = f->shape.s1;
    node->oshape.s1 = 1;
    node->oshape.s2 = 1;
    return TRUE;
}

gint32 fc_out_size(dR_Node* node) { return node->oshape.s0; }

gboolean fc_schedule(dR_Graph* net, dR_Node* node) {
    dR_FC_Data* f = fc_of(node);
    if (f->activation != tLinear && f->activation != tReLU) {
        say("FullyConnected Layer %d: activation %d is not implemented (0 linear, 1 ReLU)! \n", node->layerID, (int)f->activation);
        return FALSE;
    }
    if (debug(net)) say("Scheduled FullyConnected Layer!\n");
    return TRUE;
}

gboolean fc_allocate(dR_Graph* net, dR_Node* node) {
    dR_FC_Data* f = fc_of(node);
    const int K = f->shape.s0, N = f->shape.s1;
    if ((long long)K * N >= (1ll << 31)) { say("FullyConnected Layer %d: %dx%d weights exceed 2^31 elements! \n", node->layerID, K, N); return FALSE; }
    gboolean ok = dR_createFloatBuffer(net, &f->weightsBuf, K * N, CL_MEM_READ_ONLY);
    if (f->useBias) ok = ok && dR_createFloatBuffer(net, &f->biasBuf, N, CL_MEM_READ_ONLY);
    const size_t scratch = drhip_fc_scratch_floats(K, N);
    if (scratch > 0) ok = ok && dR_createFloatBuffer(net, &f->partialsBuf, (gint)scratch, CL_MEM_READ_WRITE);
    return ok;
}

gboolean fc_fill(dR_Graph* net, dR_Node* node) {
    dR_FC_Data* f = fc_of(node);
    if (!f->hasVariables) { say("FullyConnected Layer %d has no weights: call dR_FullyConnected_setVariables first! \n", node->layerID); return FALSE; }
    const int K = f->shape.s0, N = f->shape.s1;
    const size_t bytes = (size_t)K * N * sizeof(float);
    gboolean ok = TRUE;
    const bool flat = f->ishape.s2 == 1 || f->ishape.s0 * f->ishape.s1 == 1;    // HWC order == CHW order
    if (flat) {
        ok = dR_uploadArray(net, (gchar*)"", f->weights, 0, bytes, f->weightsBuf);
    } else {
        // The caller's rows count the input in [H][W][C] order; re-order them once to the
        // [C][H][W] order of the producer's buffer so that the GEMV reads both operands linearly.
        cl_mem raw = NULL;
        if (!dR_createFloatBuffer(net, &raw, K * N, CL_MEM_READ_ONLY)) return FALSE;
        ok = dR_uploadArray(net, (gchar*)"", f->weights, 0, bytes, raw);
        if (ok) ok = !device_failed(net, drhip_fc_permute_rows_f32((const float*)raw, (float*)f->weightsBuf, f->ishape.s0,
                                                                   f->ishape.s1, f->ishape.s2, N, stream_of(net)), "fc row permutation");
        if (ok) ok = !device_failed(net, drhip_stream_sync(stream_of(net)), "fc row permutation (sync)");
        dR_clMemoryBufferCleanup(net, raw);
        net->clConfig->memConsumptionGPU -= (glong)bytes;
    }
    if (ok && f->useBias) ok = dR_uploadArray(net, (gchar*)"", f->biases, 0, (size_t)N * sizeof(float), f->biasBuf);
    return ok;
}

// Where a node that skipped its finishing kernel left its output: an FC node its slice sums, a
// global average pooling behind a 1x1 convolution the convolution's per-tile pixel sums.
drhip_deferred_vec deferred_output_of(dR_Node* producer) {
    drhip_deferred_vec d;
    if (producer->type == tPooling) {
        dR_Node* conv = first_input(producer);
        dR_Conv2d_Data* c = (dR_Conv2d_Data*)conv->layer;
        const int P = c->ishape.s0 * c->ishape.s1;
        d.partials = (const float*)c->workspaceBuf;
        d.bias = NULL;
        d.slices = drhip_conv1x1_poolsum_slices(P);
        d.n = c->shape.s3;
        d.relu = 0;
        d.finished = producer->output ? dev_out(producer) : NULL;
        d.divisor = (float)P;
        return d;
    }
    dR_FC_Data* p = fc_of(producer);
    d.partials = (const float*)p->partialsBuf;
    d.bias = p->useBias ? (const float*)p->biasBuf : NULL;
    d.slices = drhip_fc_slices(p->shape.s0, p->shape.s1);
    d.n = p->shape.s1;
    d.relu = p->activation == tReLU;
    d.finished = producer->output ? dev_out(producer) : NULL;   // the caller reads this tensor as well
    d.divisor = 0.0f;
    return d;
}

gboolean fc_compute(dR_Graph* net, dR_Node* node) {
    dR_FC_Data* f = fc_of(node);
    drhip_deferred_vec xdef;
    if (f->drDeferredInput) xdef = deferred_output_of(f->drDeferredInput);
    int rc = drhip_fc_ex_f32(dev_out(first_input(node)), f->drDeferredInput ? &xdef : NULL, (const float*)f->weightsBuf,
                             f->useBias ? (const float*)f->biasBuf : NULL, dev_out(node), (float*)f->partialsBuf,
                             f->shape.s0, f->shape.s1, f->activation == tReLU, f->drDeferReduce, stream_of(net));
    return !device_failed(net, rc, "deepRACIN:FullyConnected");
}

gboolean fc_cleanup_buffers(dR_Graph* net, dR_Node* node) {
    dR_FC_Data* f = fc_of(node);
    gboolean ok = dR_clMemoryBufferCleanup(net, f->weightsBuf);
    if (f->useBias) ok = dR_clMemoryBufferCleanup(net, f->biasBuf) && ok;
    ok = dR_clMemoryBufferCleanup(net, f->partialsBuf) && ok;
    f->weightsBuf = f->biasBuf = f->partialsBuf = NULL;
    return ok;
}

gboolean fc_cleanup_layer(dR_Graph*, dR_Node* node) {
    dR_FC_Data* f = fc_of(node);
    if (f->hasVariables) { free(f->weights); if (f->useBias) free(f->biases); }
    free(f);
    node->layer = NULL;
    return TRUE;
}

gchar* fc_serialize(dR_Node* node, gchar* params[], gint* numParams, gfloat* variables[], gint variableSizes[], gint* numVariables) {
    dR_FC_Data* f = fc_of(node);
    const int needVars = f->useBias ? 2 : 1;
    if (*numParams < 4 || *numVariables < needVars) {
        say("SerializeNode needs space for %d parameters and %d variables!\n", 4, needVars);
        return NULL;
    }
    params[0] = fmt_dup("%d", (int)f->activation);
    params[1] = fmt_dup("%d", f->useBias ? 1 : 0);
    params[2] = fmt_dup("%d", f->shape.s0);
    params[3] = fmt_dup("%d", f->shape.s1);
    *numParams = 4;
    *numVariables = needVars;
    variableSizes[0] = f->shape.s0 * f->shape.s1;
    variables[0] = f->weights;
    if (f->useBias) { variableSizes[1] = f->shape.s1; variables[1] = f->biases; }
    return (gchar*)"FullyConnected";
}

gchar* fc_print(dR_Node* node) {
    dR_FC_Data* f = fc_of(node);
    static const char* acts[] = { "Linear", "ReLU", "Sigmoid", "Tan" };
    return fmt_dup("Fully Connected Layer: %d\n Input neurons: %d\n Output neurons: %d\n Activation: %s\n Use bias: %s\n",
                   node->layerID, f->shape.s0, f->shape.s1, acts[f->activation & 3], f->useBias ? "Yes" : "No");
}

// ================================ Softmax ========================================================

gboolean softmax_propagate(dR_Graph* net, dR_Node* node) {
    dR_Softmax_Data* s = (dR_Softmax_Data*)node->layer;
    if (node->previous_layers->length != 1 && verbose(net))
        say("Softmax Layer with id %d has %d inputs but needs 1!\n", node->layerID, node->previous_layers->length);
    dR_Node* in = first_input(node);
    if (!in) return FALSE;
    s->ishape = in->oshape;
    node->oshape = in->oshape;
    return TRUE;
}

gboolean softmax_compute(dR_Graph* net, dR_Node* node) {
    dR_Softmax_Data* s = (dR_Softmax_Data*)node->layer;
    drhip_deferred_vec xdef;
    if (s->drDeferredInput) xdef = deferred_output_of(s->drDeferredInput);
    int rc = drhip_softmax_ex_f32(dev_out(first_input(node)), s->drDeferredInput ? &xdef : NULL, dev_out(node),
                                  s->ishape.s0 * s->ishape.s1 * s->ishape.s2, stream_of(net));
    return !device_failed(net, rc, "deepRACIN:softmax");
}

gchar* softmax_serialize(dR_Node*, gchar*[], gint* numParams, gfloat*[], gint[], gint* numVariables) {
    *numParams = 0;
    *numVariables = 0;
    return (gchar*)"Softmax";
}

gchar* softmax_print(dR_Node* node) { return fmt_dup("Softmax Layer: %d\n", node->layerID); }

}  // namespace

extern "C" {

dR_Node* dR_Pooling(dR_Graph* net, dR_Node* inputLayer, dR_Shape4* sh, dR_Shape4* st, dR_PoolingType type) {
    dR_Pooling_Data* p = zalloc<dR_Pooling_Data>();
    dR_Node* n = zalloc<dR_Node>();
    p->shape = *sh;
    p->stride = *st;
    p->poolingType = type;
    n->layer = p;
    n->type = tPooling;
    n->compute = pool_compute;
    n->schedule = pool_schedule;
    n->propagateShape = pool_propagate;
    n->getRequiredOutputBufferSize = out_volume;
    n->createKernel = nothing;
    n->allocateBuffers = nothing;
    n->fillBuffers = nothing;
    n->cleanupBuffers = nothing;
    n->cleanupLayer = free_layer;
    n->serializeNode = pool_serialize;
    n->parseAppendNode = dR_pooling_parseAppendNode;
    n->printLayer = pool_print;
    link_single_input(n, inputLayer, "Pooling Layer");
    dR_appendLayer(net, n);
    return n;
}

dR_Node* dR_pooling_parseAppendNode(dR_Graph* net, dR_Node** iNodes, gint numINodes, gchar** params, gint numParams,
                                    gfloat**, gint numVariables) {
    if (numINodes != 1) { say("Parsing Error: Pooling Node needs 1 InputNodes but got %d!\n", numINodes); return NULL; }
    if (numParams != 9 || numVariables != 0) { say("Parsing Error: Pooling Node needs 9 Parameters and 0 Variables!\n"); return NULL; }
    dR_Shape4 shape = { atoi(params[1]), atoi(params[2]), atoi(params[3]), atoi(params[4]) };
    dR_Shape4 stride = { atoi(params[5]), atoi(params[6]), atoi(params[7]), atoi(params[8]) };
    return dR_Pooling(net, iNodes[0], &shape, &stride, (dR_PoolingType)atoi(params[0]));
}

dR_Node* dR_FullyConnected(dR_Graph* net, dR_Node* inputLayer, dR_Shape2* sh, dR_ActivationType acttype, gboolean useB) {
    dR_FC_Data* f = zalloc<dR_FC_Data>();
    dR_Node* n = zalloc<dR_Node>();
    f->shape = *sh;
    f->activation = acttype;
    f->useBias = useB;
    n->layer = f;
    n->type = tFullyConnected;
    n->compute = fc_compute;
    n->schedule = fc_schedule;
    n->propagateShape = fc_propagate;
    n->getRequiredOutputBufferSize = fc_out_size;
    n->createKernel = nothing;
    n->allocateBuffers = fc_allocate;
    n->fillBuffers = fc_fill;
    n->cleanupBuffers = fc_cleanup_buffers;
    n->cleanupLayer = fc_cleanup_layer;
    n->serializeNode = fc_serialize;
    n->parseAppendNode = dR_fc_parseAppendNode;
    n->setVariables = dR_FullyConnected_setVariables;
    n->printLayer = fc_print;
    link_single_input(n, inputLayer, "Fully Connected");
    dR_appendLayer(net, n);
    return n;
}

void dR_FullyConnected_setVariables(dR_Node* node, gfloat* weights, gfloat* biases) {
    dR_FC_Data* f = fc_of(node);
    if (f->hasVariables) { free(f->weights); if (f->useBias) free(f->biases); }
    f->weights = dup_floats(weights, (size_t)f->shape.s0 * f->shape.s1);
    if (f->useBias) f->biases = dup_floats(biases, (size_t)f->shape.s1);
    f->hasVariables = TRUE;
}

dR_Node* dR_fc_parseAppendNode(dR_Graph* net, dR_Node** iNodes, gint numINodes, gchar** params, gint numParams,
                               gfloat** variables, gint numVariables) {
    if (numINodes != 1) { say("Parsing Error: FullyConnected Node needs 1 InputNodes but got %d!\n", numINodes); return NULL; }
    if (numParams != 4 || numVariables < 1 || numVariables > 2) {
        say("Parsing Error: FullyConnected Node needs 4 Parameters and 1 or 2 Variables!\n");
        return NULL;
    }
    const int useBias = atoi(params[1]);
    if (useBias && numVariables < 2) { say("Parsing Error: FullyConnected Node uses a bias but has no bias variable!\n"); return NULL; }
    dR_Shape2 shape = { atoi(params[2]), atoi(params[3]) };
    if (!parsed_var_has(0, (size_t)shape.s0 * shape.s1, "FullyConnected weights")) return NULL;
    if (useBias && !parsed_var_has(1, (size_t)shape.s1, "FullyConnected biases")) return NULL;
    dR_Node* n = dR_FullyConnected(net, iNodes[0], &shape, (dR_ActivationType)atoi(params[0]), useBias);
    dR_FullyConnected_setVariables(n, variables[0], useBias ? variables[1] : NULL);
    return n;
}

dR_Node* dR_Softmax(dR_Graph* net, dR_Node* inputLayer) {
    dR_Softmax_Data* s = zalloc<dR_Softmax_Data>();
    dR_Node* n = zalloc<dR_Node>();
    n->layer = s;
    n->type = tSoftmax;
    n->compute = softmax_compute;
    n->schedule = nothing;
    n->propagateShape = softmax_propagate;
    n->getRequiredOutputBufferSize = out_volume;
    n->createKernel = nothing;
    n->allocateBuffers = nothing;
    n->fillBuffers = nothing;
    n->cleanupBuffers = nothing;
    n->cleanupLayer = free_layer;
    n->serializeNode = softmax_serialize;
    n->parseAppendNode = dR_softmax_parseAppendNode;
    n->printLayer = softmax_print;
    link_single_input(n, inputLayer, "Softmax Layer");
    dR_appendLayer(net, n);
    return n;
}

dR_Node* dR_softmax_parseAppendNode(dR_Graph* net, dR_Node** iNodes, gint numINodes, gchar**, gint numParams, gfloat**,
                                    gint numVariables) {
    if (numINodes != 1) { say("Parsing Error: Softmax Node needs 1 InputNodes but got %d!\n", numINodes); return NULL; }
    if (numParams != 0 || numVariables != 0) { say("Parsing Error: Softmax Node needs 0 Parameters and 0 Variables!\n"); return NULL; }
    return dR_Softmax(net, iNodes[0]);
}

}  // extern "C"
