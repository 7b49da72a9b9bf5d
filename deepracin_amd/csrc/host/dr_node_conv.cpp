// Conv2d node: constructor, graph.dr (de)serialisation, and the three gfx950 execution paths.
//
// Node contract = reference src/dR_nodes_conv2d.c:12-256 (constructor, shape rule out = in/stride,
// 10 parameters + 1..2 variables in graph.dr, deep copy in setVariables).  What differs is below the
// vtable: schedule() assigns a HIP kernel variant instead of OpenCL work sizes, fillBuffers() uploads
// weights in the layout that kernel streams best, compute() enqueues through drhip_*.
#include "dr_internal.hpp"

#include <vector>

using namespace dr;

namespace {

inline dR_Conv2d_Data* conv_of(dR_Node* n) { return (dR_Conv2d_Data*)n->layer; }
inline int weight_count(const dR_Conv2d_Data* c) { return c->shape.s0 * c->shape.s1 * c->shape.s2 * c->shape.s3; }

gboolean conv_propagate(dR_Graph* net, dR_Node* node) {
    dR_Conv2d_Data* c = conv_of(node);
    if (node->previous_layers->length != 1 && verbose(net))
        say("Conv2d Layer with id %d has %d inputs but needs 1!\n", node->layerID, node->previous_layers->length);
    dR_Node* in = first_input(node);
    if (!in) return FALSE;
    c->ishape = in->oshape;
    if (c->stride.s1 <= 0 || c->stride.s2 <= 0) { say("Conv2d stride must be positive! \n"); return FALSE; }
    node->oshape.s0 = c->ishape.s0 / c->stride.s1;
    node->oshape.s1 = c->ishape.s1 / c->stride.s2;
    node->oshape.s2 = c->shape.s3;
    if (node->oshape.s0 <= 0 || node->oshape.s1 <= 0 || node->oshape.s2 <= 0) {
        say("Conv2d shape propagates to Zero. False shape parameters! \n");
        return FALSE;
    }
    if (c->ishape.s2 != c->shape.s2) {
        say("Conv2d Layer %d expects %d input channels but its input has %d! \n", node->layerID, c->shape.s2, c->ishape.s2);
        return FALSE;
    }
    return TRUE;
}

gint32 conv_out_size(dR_Node* node) { return node->oshape.s0 * node->oshape.s1 * node->oshape.s2; }

gchar* conv_serialize(dR_Node* node, gchar* params[], gint* numParams, gfloat* variables[], gint variableSizes[],
                      gint* numVariables) {
    dR_Conv2d_Data* c = conv_of(node);
    const int needVars = c->useBias ? 2 : 1;
    if (*numParams < 10 || *numVariables < needVars) {
        say("SerializeNode needs space for %d parameters and %d variables!\n", 10, needVars);
        return NULL;
    }
    const int vals[10] = { (int)c->activation, c->useBias ? 1 : 0, c->shape.s0, c->shape.s1, c->shape.s2, c->shape.s3,
                           c->stride.s0, c->stride.s1, c->stride.s2, c->stride.s3 };
    for (int i = 0; i < 10; ++i) params[i] = fmt_dup("%d", vals[i]);
    *numParams = 10;
    *numVariables = needVars;
    variableSizes[0] = weight_count(c);
    variables[0] = c->weights;
    if (c->useBias) { variableSizes[1] = c->shape.s3; variables[1] = c->biases; }
    return (gchar*)"Conv2D";
}

gchar* conv_print(dR_Node* node) {
    dR_Conv2d_Data* c = conv_of(node);
    static const char* acts[] = { "Linear", "ReLU", "Sigmoid", "Tan" };
    static const char* algos[] = { "direct", "Winograd F(2x2,3x3) MFMA", "1x1 MFMA GEMM" };
    return fmt_dup("Conv2d Layer: %d\n Filter dimensions: %dx%d\n Input channels: %d\n Output channels: %d\n"
                   " Activation: %s\n Stride: %d, %d, %d, %d\n Use bias: %s\n Kernel: %s (variant %d)\n",
                   node->layerID, c->shape.s0, c->shape.s1, c->shape.s2, c->shape.s3, acts[c->activation & 3],
                   c->stride.s0, c->stride.s1, c->stride.s2, c->stride.s3, c->useBias ? "Yes" : "No",
                   algos[c->algo], c->variant);
}

// ---- schedule: kernel variant and tile parameters for gfx950 -------------------------------------
gboolean conv_schedule(dR_Graph* net, dR_Node* node) {
    dR_Conv2d_Data* c = conv_of(node);
    const int W = c->ishape.s0, H = c->ishape.s1, I = c->shape.s2, O = c->shape.s3;
    // The matrix-core convolution kernels carry W, H, I and O in 16-bit fields of their packed arguments;
    // a layer beyond that takes the general direct kernel.
    // They also address their input and their filters with 32-bit byte offsets (the entry points refuse 2^29 input
    // elements or more); such a layer takes the general direct kernel, which indexes with size_t, as well.
    const bool packable = W <= 65535 && H <= 65535 && I <= 65535 && O <= 65535 && (long long)W * H * I < (1ll << 29) &&
                          (long long)W * H * O < (1ll << 31) && (long long)(I + 7) * (O + 31) * 16 < (1ll << 29);
    if (c->algo == drConvWinograd && !packable) c->algo = drConvDirect;
    switch (c->algo) {
        case drConvWinograd: c->variant = drhip_conv3x3_winograd_pick_variant(W, H, I, O); break;
        case drConv1x1Gemm:  c->variant = drhip_conv1x1_pick_variant(W * H, I, O); break;
        default: {
            // 3x3, stride 1 or 2, more than 4 input channels: the implicit GEMM on the matrix cores over a filter
            // bank laid out at prepare time; everything else: the direct launcher sizes its own tiles
            const char* valu = getenv("DR_DIRECT_VALU");
            c->drDirectBank = packable && c->shape.s0 == 3 && c->shape.s1 == 3 && I > 4 && c->stride.s1 == c->stride.s2 &&
                              (c->stride.s1 == 1 || c->stride.s1 == 2) && !(valu && strcmp(valu, "1") == 0);
            c->variant = c->drDirectBank ? drhip_conv3x3_direct_pick_variant(W / c->stride.s1, H / c->stride.s2, I, O) : 0;
            break;
        }
    }
    if ((c->shape.s0 & 1) == 0 || (c->shape.s1 & 1) == 0) {
        say("Conv2d Layer %d: filter %dx%d must have odd side lengths! \n", node->layerID, c->shape.s0, c->shape.s1);
        return FALSE;
    }
    if (c->activation != tLinear && c->activation != tReLU) {
        say("Conv2d Layer %d: activation %d is not implemented (0 linear, 1 ReLU)! \n", node->layerID, (int)c->activation);
        return FALSE;
    }
    if (debug(net)) say("Scheduled Conv2D Layer %d: algo %d variant %d\n", node->layerID, (int)c->algo, c->variant);
    return TRUE;
}

gboolean conv_create_kernel(dR_Graph*, dR_Node*) { return TRUE; }   // kernels are built into the library

// Output channels the node's launch produces: its own plus those of an absorbed 1x1 sibling.
inline int launch_channels(const dR_Conv2d_Data* c) {
    return c->shape.s3 + (c->drAbsorbed1x1 ? conv_of(c->drAbsorbed1x1)->shape.s3 : 0);
}
inline bool launch_has_bias(const dR_Conv2d_Data* c) {
    return c->useBias || (c->drAbsorbed1x1 && conv_of(c->drAbsorbed1x1)->useBias);
}

gboolean conv_allocate(dR_Graph* net, dR_Node* node) {
    dR_Conv2d_Data* c = conv_of(node);
    if (c->drAbsorbedBy) return TRUE;           // the 3x3 sibling carries this node's filters and bias
    const bool wino = c->algo == drConvWinograd;
    const int O = launch_channels(c);
    if (c->drAbsorbed1x1)                       // the joint layer is wider than the one schedule() saw
        c->variant = drhip_conv3x3_winograd_pick_variant(c->ishape.s0, c->ishape.s1, c->shape.s2, O);
    const int n = wino ? (int)drhip_conv3x3_winograd_filter_floats(c->shape.s2, O)
                       : c->drDirectBank ? (int)drhip_conv3x3_direct_filter_floats(c->shape.s2, O) : weight_count(c);
    gboolean ok = dR_createFloatBuffer(net, &c->weightsBuf, n, CL_MEM_READ_ONLY);
    if (launch_has_bias(c)) ok = ok && dR_createFloatBuffer(net, &c->biasBuf, O, CL_MEM_READ_ONLY);
    const size_t ws = wino ? drhip_conv3x3_winograd_workspace_floats(c->ishape.s0, c->ishape.s1, c->shape.s2, O, c->variant) : 0;
    if (ws > 0) ok = ok && dR_createFloatBuffer(net, &c->workspaceBuf, (gint)ws, CL_MEM_READ_WRITE);   // split-K partial tiles
    if (c->drFusedAvgPool)                      // per-tile pixel sums for the pooling behind this layer
        ok = ok && dR_createFloatBuffer(net, &c->workspaceBuf, drhip_conv1x1_poolsum_slices(c->ishape.s0 * c->ishape.s1) * O, CL_MEM_READ_WRITE);
    return ok;
}

gboolean conv_fill(dR_Graph* net, dR_Node* node) {
    dR_Conv2d_Data* c = conv_of(node);
    if (!c->hasVariables) { say("Conv2d Layer %d has no weights: call dR_Conv2d_setVariables first! \n", node->layerID); return FALSE; }
    if (c->drAbsorbedBy) return TRUE;
    gboolean ok = TRUE;
    if (c->algo == drConvWinograd) {
        // raw weights go up once, U = G g G^T is produced on the device, the raw copy is dropped.
        // With an absorbed 1x1 sibling the joint filter bank is [I][O1 + O3][3][3]: the sibling's
        // channels first (they sit just below this node's in the concat), centre tap only.
        const dR_Conv2d_Data* a = c->drAbsorbed1x1 ? conv_of(c->drAbsorbed1x1) : NULL;
        if (a && !a->hasVariables) { say("Conv2d Layer %d has no weights: call dR_Conv2d_setVariables first! \n", c->drAbsorbed1x1->layerID); return FALSE; }
        const int I = c->shape.s2, O3 = c->shape.s3, O1 = a ? a->shape.s3 : 0, O = O1 + O3;
        std::vector<float> joint;
        const float* host = c->weights;
        if (a) {
            joint.assign((size_t)I * O * 9, 0.0f);
            for (int i = 0; i < I; ++i) {
                for (int o = 0; o < O1; ++o) joint[((size_t)i * O + o) * 9 + 4] = a->weights[(size_t)i * O1 + o];
                memcpy(&joint[((size_t)i * O + O1) * 9], &c->weights[(size_t)i * O3 * 9], (size_t)O3 * 9 * sizeof(float));
            }
            host = joint.data();
        }
        const size_t rawBytes = (size_t)I * O * 9 * sizeof(float);
        cl_mem raw = NULL;
        if (!dR_createFloatBuffer(net, &raw, I * O * 9, CL_MEM_READ_ONLY)) return FALSE;
        ok = dR_uploadArray(net, (gchar*)"", (void*)host, 0, rawBytes, raw);
        if (ok) ok = !device_failed(net, drhip_winograd_filter_transform_f32((const float*)raw, (float*)c->weightsBuf, I, O, stream_of(net)),
                                    "winograd filter transform");
        if (ok) ok = !device_failed(net, drhip_stream_sync(stream_of(net)), "winograd filter transform (sync)");
        dR_clMemoryBufferCleanup(net, raw);
        net->clConfig->memConsumptionGPU -= (glong)rawBytes;
        if (ok && c->workspaceBuf && (c->variant & 0x800))     // joined splits recognise missing partial tiles by a marker
            ok = !device_failed(net, drhip_conv3x3_winograd_workspace_prepare_f32(
                                         (float*)c->workspaceBuf, drhip_conv3x3_winograd_workspace_floats(c->ishape.s0, c->ishape.s1, I, O, c->variant),
                                         stream_of(net)), "winograd workspace");
        if (ok && a && launch_has_bias(c)) {
            std::vector<float> bias((size_t)O, 0.0f);
            if (a->useBias) memcpy(bias.data(), a->biases, (size_t)O1 * sizeof(float));
            if (c->useBias) memcpy(bias.data() + O1, c->biases, (size_t)O3 * sizeof(float));
            return dR_uploadArray(net, (gchar*)"", bias.data(), 0, (size_t)O * sizeof(float), c->biasBuf);
        }
    } else if (c->drDirectBank) {
        // raw weights go up once, the filter bank is laid out on the device, the raw copy is dropped
        const int I = c->shape.s2, O = c->shape.s3;
        const size_t rawBytes = (size_t)weight_count(c) * sizeof(float);
        cl_mem raw = NULL;
        if (!dR_createFloatBuffer(net, &raw, weight_count(c), CL_MEM_READ_ONLY)) return FALSE;
        ok = dR_uploadArray(net, (gchar*)"", c->weights, 0, rawBytes, raw);
        if (ok) ok = !device_failed(net, drhip_conv3x3_direct_filter_layout_f32((const float*)raw, (float*)c->weightsBuf, I, O, stream_of(net)),
                                    "direct filter layout");
        if (ok) ok = !device_failed(net, drhip_stream_sync(stream_of(net)), "direct filter layout (sync)");
        dR_clMemoryBufferCleanup(net, raw);
        net->clConfig->memConsumptionGPU -= (glong)rawBytes;
    } else {
        ok = dR_uploadArray(net, (gchar*)"", c->weights, 0, (size_t)weight_count(c) * sizeof(float), c->weightsBuf);
    }
    if (ok && c->useBias) ok = dR_uploadArray(net, (gchar*)"", c->biases, 0, (size_t)c->shape.s3 * sizeof(float), c->biasBuf);
    return ok;
}

gboolean conv_compute(dR_Graph* net, dR_Node* node) {
    dR_Conv2d_Data* c = conv_of(node);
    if (c->drAbsorbedBy) return TRUE;           // computed by the 3x3 sibling's launch
    dR_Node* src = first_input(node);
    const float* in = dev_out(src);
    // with drFusedPool this is the pooling node's buffer; with an absorbed 1x1 sibling the launch
    // starts at that sibling's channels, which lie directly below this node's in the concat buffer
    float* out = c->drAbsorbed1x1 ? dev_out(c->drAbsorbed1x1) : dev_out(node);
    const float* w = (const float*)c->weightsBuf;
    const float* b = launch_has_bias(c) ? (const float*)c->biasBuf : NULL;
    const int W = c->ishape.s0, H = c->ishape.s1, I = c->shape.s2, O = launch_channels(c);
    const int relu = c->activation == tReLU;
    int rc;
    switch (c->algo) {
        case drConvWinograd:
            rc = drhip_conv3x3_winograd_f32(in, w, b, out, W, H, I, O,
                                            (relu ? DRHIP_EPILOGUE_RELU : 0) | (c->drFusedPool ? DRHIP_EPILOGUE_MAXPOOL2 : 0),
                                            c->variant, (float*)c->workspaceBuf, stream_of(net));
            break;
        case drConv1x1Gemm:
            if (c->drFusedAvgPool)
                rc = drhip_conv1x1_poolsum_f32(in, w, b, (float*)c->workspaceBuf, W * H, I, O, relu, stream_of(net));
            else if (c->drPooledInput) {        // the 3x3/2 max pooling in front is taken while loading its input
                const dR_Pooling_Data* pd = (const dR_Pooling_Data*)c->drPooledInput->layer;
                rc = drhip_conv1x1_pooled3s2_f32(dev_out(first_input(c->drPooledInput)), w, b, out, pd->ishape.s0, pd->ishape.s1,
                                                 I, O, relu, stream_of(net));
            } else
                rc = drhip_conv1x1_f32(in, w, b, out, W * H, I, O, relu, c->variant, stream_of(net));
            break;
        default:
            if (c->drFusedPool)                 // first layer + the 3x3/2 max pool behind it (out = the pool's buffer)
                rc = drhip_conv3x3_pool3s2_f32(in, w, b, out, W, H, I, O, c->stride.s1, c->stride.s2, relu, stream_of(net));
            else if (c->drDirectBank)
                rc = drhip_conv3x3_direct_mfma_f32(in, w, b, out, W, H, I, O, c->stride.s1, relu, c->variant, stream_of(net));
            else
                rc = drhip_conv2d_direct_f32(in, w, b, out, W, H, I, O, c->shape.s0, c->shape.s1,
                                             c->stride.s1, c->stride.s2, relu, stream_of(net));
            break;
    }
    return !device_failed(net, rc, "deepRACIN:conv2d");
}

gboolean conv_cleanup_buffers(dR_Graph* net, dR_Node* node) {
    dR_Conv2d_Data* c = conv_of(node);
    gboolean ok = dR_clMemoryBufferCleanup(net, c->weightsBuf);
    ok = dR_clMemoryBufferCleanup(net, c->biasBuf) && ok;
    ok = dR_clMemoryBufferCleanup(net, c->workspaceBuf) && ok;
    c->weightsBuf = c->biasBuf = c->workspaceBuf = NULL;
    return ok;
}

gboolean conv_cleanup_layer(dR_Graph*, dR_Node* node) {
    dR_Conv2d_Data* c = conv_of(node);
    if (c->hasVariables) { free(c->weights); if (c->useBias) free(c->biases); }
    free(c);
    node->layer = NULL;
    return TRUE;
}

}  // namespace

extern "C" {

dR_Node* dR_Conv2d(dR_Graph* net, dR_Node* inputLayer, dR_Shape4* sh, dR_Shape4* st, dR_ActivationType acttype,
                   gboolean useB) {
    dR_Conv2d_Data* c = zalloc<dR_Conv2d_Data>();
    dR_Node* n = zalloc<dR_Node>();
    c->shape = *sh;
    c->stride = *st;
    c->activation = acttype;
    c->useBias = useB;
    c->winogradn = 2;
    n->layer = c;
    n->type = tConv2d;

    // Same dispatch rule as the reference (src/dR_nodes_conv2d.c:37-81), plus an override for
    // benchmarking the direct kernel on a layer Winograd would normally take.
    const bool unitStride = st->s1 == 1 && st->s2 == 1;
    const char* force = getenv("DR_CONV3X3");
    if (sh->s0 == 3 && sh->s1 == 3 && unitStride && !(force && strcmp(force, "direct") == 0)) c->algo = drConvWinograd;
    else if (sh->s0 == 1 && sh->s1 == 1 && unitStride) c->algo = drConv1x1Gemm;
    else c->algo = drConvDirect;

    n->compute = conv_compute;
    n->schedule = conv_schedule;
    n->propagateShape = conv_propagate;
    n->getRequiredOutputBufferSize = conv_out_size;
    n->createKernel = conv_create_kernel;
    n->allocateBuffers = conv_allocate;
    n->fillBuffers = conv_fill;
    n->cleanupBuffers = conv_cleanup_buffers;
    n->cleanupLayer = conv_cleanup_layer;
    n->printLayer = conv_print;
    n->serializeNode = conv_serialize;
    n->parseAppendNode = dR_conv2d_parseAppendNode;
    n->setVariables = dR_Conv2d_setVariables;
    n->generateKernel = NULL;
    n->createKernelName = NULL;

    link_single_input(n, inputLayer, "Conv2d");
    dR_appendLayer(net, n);
    return n;
}

void dR_Conv2d_setVariables(dR_Node* node, gfloat* weights, gfloat* biases) {
    dR_Conv2d_Data* c = conv_of(node);
    if (c->hasVariables) { free(c->weights); if (c->useBias) free(c->biases); }
    c->weights = dup_floats(weights, (size_t)weight_count(c));
    if (c->useBias) c->biases = dup_floats(biases, (size_t)c->shape.s3);
    c->hasVariables = TRUE;
}

dR_Node* dR_conv2d_parseAppendNode(dR_Graph* net, dR_Node** iNodes, gint numINodes, gchar** params, gint numParams,
                                   gfloat** variables, gint numVariables) {
    if (numINodes != 1) { say("Parsing Error: Conv2d Node needs 1 InputNodes but got %d!\n", numINodes); return NULL; }
    if (numParams != 10 || numVariables < 1 || numVariables > 2) {
        say("Parsing Error: Conv2d Node needs 10 Parameters and 1 or 2 Variables!\n");
        return NULL;
    }
    const int useBias = atoi(params[1]);
    if (useBias && numVariables < 2) { say("Parsing Error: Conv2d Node uses a bias but has no bias variable!\n"); return NULL; }
    dR_Shape4 shape = { atoi(params[2]), atoi(params[3]), atoi(params[4]), atoi(params[5]) };
    dR_Shape4 stride = { atoi(params[6]), atoi(params[7]), atoi(params[8]), atoi(params[9]) };
    if (!parsed_var_has(0, (size_t)shape.s0 * shape.s1 * shape.s2 * shape.s3, "Conv2d weights")) return NULL;
    if (useBias && !parsed_var_has(1, (size_t)shape.s3, "Conv2d biases")) return NULL;
    dR_Node* n = dR_Conv2d(net, iNodes[0], &shape, &stride, (dR_ActivationType)atoi(params[0]), useBias);
    dR_Conv2d_setVariables(n, variables[0], useBias ? variables[1] : NULL);
    return n;
}

}  // extern "C"
