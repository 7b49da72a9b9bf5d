/*
 * dR_nodes.h -- node constructors and per-node data of the CNN layer path.
 *
 * Constructor names, argument order and meaning are those of the reference
 * (include/dR_nodes_conv2d.h:70,86; dR_nodes_pooling.h:28; dR_nodes_fc.h:30,32;
 *  dR_nodes_math.h:122,189; dR_nodes_transform.h:23,100).  The *_Data structs keep the reference's
 * semantic fields (shape, stride, weights, useBias ...) and replace the OpenCL work-size fields by
 * the gfx950 launch plan that schedule() fills in.
 */
#ifndef DR_NODES_H
#define DR_NODES_H

#include "dR_types.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ================================ Conv2d ====================================================== */

/* Algorithms the gfx950 scheduler can pick for a Conv2d node. */
enum dR_ConvAlgo {
    drConvDirect   = 0,     /* register-tiled direct correlation, any odd k, any stride (VALU) */
    drConvWinograd = 1,     /* fused F(2x2,3x3), 16 batched fp32-MFMA GEMMs */
    drConv1x1Gemm  = 2      /* fp32-MFMA GEMM over [I][H*W] */
};
typedef enum dR_ConvAlgo dR_ConvAlgo;

typedef struct dR_Conv2d_Data dR_Conv2d_Data;
struct dR_Conv2d_Data {
    dR_Shape3           ishape;         /* input (W,H,C) */
    dR_Shape4           shape;          /* (kw, kh, I, O) */
    dR_Shape4           stride;         /* (1, sx, sy, 1) */
    gfloat*             weights;        /* host copy, [I][O][kh][kw] */
    gfloat*             biases;         /* host copy, [O] */
    cl_mem              weightsBuf;     /* device: direct/1x1 -> [I][O][kh][kw]; Winograd -> transformed filters U */
    cl_mem              biasBuf;
    gboolean            useBias;
    gboolean            hasVariables;
    dR_ActivationType   activation;
    /* gfx950 launch plan (filled by schedule()) */
    dR_ConvAlgo         algo;
    gint                variant;        /* tile configuration id understood by the drhip_* launcher */
    gint                winogradn;      /* always 2: F(2x2,3x3) */
    cl_mem              workspaceBuf;   /* split-K scratch of the Winograd kernel, NULL when the layer is not split */
    dR_Node*            drAbsorbed1x1;  /* set by the buffer planner on a Winograd node: the 1x1 sibling (same input, the channels
                                           just below this node's in a fused concat) whose filters ride along as centre taps */
    dR_Node*            drAbsorbedBy;   /* set on that 1x1 sibling: its compute() launches nothing */
    gboolean            drFusedAvgPool; /* set by the buffer planner: a 1x1 layer whose only consumer is a global average
                                           pooling read by an FC or softmax node; the layer leaves per-tile pixel sums
                                           in workspaceBuf and neither its tensor nor the pooled one is computed by a kernel of its own */
    gboolean            drFusedPool;    /* set by the buffer planner: the node's only consumer is a 2x2/2 max pool and
                                           this node writes the pooled tensor straight into that node's buffer */
    gboolean            drDirectBank;   /* set by schedule() on a direct 3x3 layer with more than 4 input channels and stride
                                           1 or 2: weightsBuf holds the filter bank of the matrix-core kernel, variant its tiles */
    dR_Node*            drPooledInput;  /* set by the buffer planner on a 1x1 layer whose input is a 3x3/2 max pooling
                                           read by nobody else: that pooling node; the layer reads the pooling's own
                                           input and takes the window maxima while loading, the pooling launches nothing */
};

/*
 * Append a 2-D convolution.  filtershape = (kw, kh, I, O); stride = (1, sx, sy, 1).
 * out[o,y,x] = act(b[o] + sum_{c,j,i} in[c, y*sy+j, x*sx+i] * w[c][o][j+kh/2][i+kw/2]),
 * j in [-kh/2,kh/2], i in [-kw/2,kw/2], zero padding; output (W/sx, H/sy, O) (floor).
 * Dispatch (reference src/dR_nodes_conv2d.c:37-81): 3x3 stride 1 -> Winograd F(2x2,3x3),
 * 1x1 stride 1 -> 1x1 GEMM, otherwise direct.  The environment variable DR_CONV3X3=direct forces
 * the direct kernel for 3x3 stride-1 nodes created afterwards (the reference has no such switch).
 */
dR_Node* dR_Conv2d(dR_Graph* net, dR_Node* inputnode, dR_Shape4* filtershape, dR_Shape4* stride,
                   dR_ActivationType activation, gboolean useBias);
/* Deep-copies weights [I][O][kh][kw] and biases [O] (biases may be NULL when useBias is FALSE). */
void     dR_Conv2d_setVariables(dR_Node* node, gfloat* weights, gfloat* biases);

/* ================================ Pooling ===================================================== */

enum dR_PoolingType { tMax, tAverage, tl2norm /* unimplemented upstream and here */ };
typedef enum dR_PoolingType dR_PoolingType;

typedef struct dR_Pooling_Data dR_Pooling_Data;
struct dR_Pooling_Data {
    dR_Shape3       ishape;
    dR_Shape4       shape;      /* (ignored, sx, sy, sz) */
    dR_Shape4       stride;     /* (ignored, stx, sty, stz) */
    dR_PoolingType  poolingType;
    gchar**         shaderSrc;  /* unused placeholder */
    gboolean        useLMEM;    /* unused placeholder */
    gboolean        drFused;    /* set by the buffer planner: the producing convolution already pooled; compute() is a no-op */
};

/* Output dims = ceil(in/stride); window anchored top-left at (x*stx, y*sty, z*stz), no leading
 * pad, samples beyond the input read 0.0f (reference src/dR_nodes_pooling.c:186-224, 277-401). */
dR_Node* dR_Pooling(dR_Graph* net, dR_Node* inputLayer, dR_Shape4* shape, dR_Shape4* stride,
                    dR_PoolingType poolingtype);

/* ================================ FullyConnected ============================================== */

typedef struct dR_FC_Data dR_FC_Data;
struct dR_FC_Data {
    dR_Shape3           ishape;
    dR_Shape2           shape;          /* (K inputs, N outputs) */
    gfloat*             weights;        /* host copy [K][N], n fastest; k counts the input in [H][W][C] order */
    gfloat*             biases;
    cl_mem              weightsBuf;     /* device [K][N] with rows re-ordered to the [C][H][W] buffer order */
    cl_mem              biasBuf;
    gboolean            useBias;
    gboolean            hasVariables;
    dR_ActivationType   activation;
    /* gfx950 plan */
    cl_mem              partialsBuf;    /* split-K partial sums, NULL when the layer is not split */
    gboolean            drDeferReduce;  /* set by the buffer planner: the only consumer (FC or softmax) sums the partials itself */
    dR_Node*            drDeferredInput; /* set by the buffer planner: the FC node in front left its output as partial sums */
};

/* y[n] = act(b[n] + sum_k x_hwc[k] * W[k][n]); shape = (K, N); K must equal W*H*C of the input. */
dR_Node* dR_FullyConnected(dR_Graph* net, dR_Node* inputLayer, dR_Shape2* shape,
                           dR_ActivationType activation, gboolean useBias);
void     dR_FullyConnected_setVariables(dR_Node* layer, gfloat* weights, gfloat* bias);

/* ================================ Softmax ===================================================== */

typedef struct dR_Softmax_Data dR_Softmax_Data;
struct dR_Softmax_Data {
    dR_Shape3   ishape;
    cl_kernel   clKernelComputeExp;     /* unused placeholder */
    gfloat*     expsHost;               /* unused placeholder: the sum stays on the device */
    dR_Node*    drDeferredInput;        /* set by the buffer planner: the FC node in front left its output as partial sums */
};

/* p = exp(x) / sum(exp(x)) over all W*H*C elements of the input. */
dR_Node* dR_Softmax(dR_Graph* net, dR_Node* inputLayer);

/* ================================ Concat / Slice ============================================== */

typedef struct dR_Concat_Data dR_Concat_Data;
struct dR_Concat_Data {
    gint        n;
    gint        concatDim;                  /* 0 = W, 1 = H, 2 = C */
    gint        maxInputSizeInConcatDim;
    gint*       inputSizesInConcatDim;
    gboolean    drFused;                    /* TRUE: producers write straight into this node's buffer */
};

/* Concatenate n (2..3) inputs along concatDim.  When concatDim == 2 and every input is produced
 * for this node alone, the buffer planner lets the producers write at their channel offset of the
 * concat buffer and compute() launches nothing. */
dR_Node* dR_Concat(dR_Graph* net, dR_Node** inputNodes, gint n, gint concatDim);

typedef struct dR_Slice_Data dR_Slice_Data;
struct dR_Slice_Data {
    dR_Shape4   ishape;     /* input (W,H,C,-) */
    dR_Shape4   origin;     /* first element of the box (x,y,z,-) */
    dR_Shape4   oshape;     /* box extent (w,h,c,-) */
};

/* out[z][y][x] = in[z+origin.s2][y+origin.s1][x+origin.s0] for a (shape.s0,shape.s1,shape.s2) box. */
dR_Node* dR_Slice(dR_Graph* net, dR_Node* inputLayer, dR_Shape4* origin, dR_Shape4* shape);

/* ================================ element-wise scalar op ====================================== */

enum dR_ElemWise1OperationType { tAddS, tSubS, tMulS, tDivS, tLog, tExp, tSqrt, tFill, tPowS };
typedef enum dR_ElemWise1OperationType dR_ElemWise1OperationType;

typedef struct dR_ElemWise1Op_Data dR_ElemWise1Op_Data;
struct dR_ElemWise1Op_Data {
    dR_Shape3                   ishape;
    dR_ElemWise1OperationType   op;
    gfloat                      scalar;
};

dR_Node* dR_ElemWise1Operation(dR_Graph* net, dR_Node* inputNode, dR_ElemWise1OperationType op,
                               gfloat scalar);

/* ================================ normalization =============================================== */

/* Same numbering as the reference (include/dR_nodes_misc.h:268-272). */
enum dR_NormalizationType { tNormMean, tNormDev, tNormMeanDev };
typedef enum dR_NormalizationType dR_NormalizationType;

typedef struct dR_Normalization_Data dR_Normalization_Data;
struct dR_Normalization_Data {
    dR_Shape3               ishape;
    dR_NormalizationType    type;
    gfloat                  targetMean;
    gfloat                  targetDev;
    cl_mem                  tempFloatBuffer1;   /* per-workgroup partial sums of both reductions */
    cl_mem                  tempFloatBuffer2;   /* unused placeholder (the reference ping-pongs between two) */
};

/* Shift and/or scale the whole input tensor to a target mean / standard deviation taken over all
 * W*H*C elements (population deviation about the mean): tNormMean y = x + (targetMean - mean),
 * tNormDev y = x * (targetDev / dev), tNormMeanDev both (reference src/dR_nodes_misc.c:1051-1446;
 * graph.dr: "Normalization", params `type targetMean targetDev`). */
dR_Node* dR_Normalization(dR_Graph* net, dR_Node* inputLayer, dR_NormalizationType type, gfloat targetMean,
                          gfloat targetDev);

/* ================================ nodes outside the CNN layer path ============================ */

/* The reference's Python wrapper binds these constructors when it is imported
 * (python/deepracin/__init__.py.in:146-211), so the symbols exist with the reference's signatures
 * (include/dR_nodes_filter.h:61,63,161; dR_nodes_math.h:45; dR_nodes_misc.h:40,102,167,230;
 * dR_nodes_transform.h:168).  The node types themselves (image filters, two-tensor arithmetic,
 * region-of-interest, colour, upscaling, label and crop nodes) are not part of this build: every
 * constructor prints which node type was asked for, appends nothing and returns NULL, and
 * dR_MaskDependentFilter_setVariables does nothing. */
enum dR_ElemWise2OperationType { tAdd, tSub, tMul, tDiv, tPow };
typedef enum dR_ElemWise2OperationType dR_ElemWise2OperationType;
enum dR_UpscalingType { tNearestNUp, tLinearUp, tBicubicUp };
typedef enum dR_UpscalingType dR_UpscalingType;
enum dR_LabelCreationType { t3to2ClassesBin, t3to2ClassesConf, t2ClassesBin, t2ClassesConf, tnClasses };
typedef enum dR_LabelCreationType dR_LabelCreationType;

dR_Node* dR_MaskDependentFilter(dR_Graph* net, dR_Node* inputImage, dR_Node* inputFilterMask, dR_Shape3* shape);
void     dR_MaskDependentFilter_setVariables(dR_Node* layer, gfloat* weights, gfloat* bias);
dR_Node* dR_PerPixelFilter(dR_Graph* net, dR_Node* inputImage, dR_Node* inputFilter, dR_Shape4* shape, dR_Shape4* stride);
dR_Node* dR_ElemWise2Operation(dR_Graph* net, dR_Node* inputNode1, dR_Node* inputNode2, dR_ElemWise2OperationType op);
dR_Node* dR_ResolveRoI(dR_Graph* net, dR_Node* inputLayer, dR_Shape3* shape);
dR_Node* dR_RGB2gray(dR_Graph* net, dR_Node* inputLayer);
dR_Node* dR_Upscaling(dR_Graph* net, dR_Node* inputLayer, dR_UpscalingType type, gint scaleFactorX, gint scaleFactorY);
dR_Node* dR_LabelCreation(dR_Graph* net, dR_Node* inputLayer, dR_LabelCreationType type, gfloat class0offset,
                          gfloat class1offset, gfloat class2offset);
dR_Node* dR_CropOrPad(dR_Graph* net, dR_Node* inputLayer, dR_Shape3* targetshape);
/* Looked up only when the wrapper's Conv2dTransposed() is called (include/dR_nodes_conv2d.h:229,245;
 * shapes by value there); the node is unfinished in the reference. */
dR_Node* dR_Conv2dTransposed(dR_Graph* net, dR_Node* inputnode, dR_Shape4 filtershape, dR_Shape4 stride,
                             dR_ActivationType activation, gboolean useBias);
void     dR_Conv2dtransposed_setVariables(dR_Node* node, gfloat* weights, gfloat* biases);

#ifdef __cplusplus
}
#endif
#endif /* DR_NODES_H */
