/* dR_nodes_pooling.h -- kept so that sources including the reference's header of this name still compile.
 * In this build every declaration lives in deepRACIN.h (graph API, core, device-memory helpers)
 * and dR_nodes.h (node constructors). */
#ifndef DR_NODES_POOLING_FWD_H
#define DR_NODES_POOLING_FWD_H
#include "deepRACIN.h"
#endif
