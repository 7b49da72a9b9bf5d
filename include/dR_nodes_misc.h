/* dR_nodes_misc.h -- kept so that sources including the reference's header of this name still compile.
 * In this build every declaration lives in deepRACIN.h (graph API, core, device-memory helpers)
 * and dR_nodes.h (node constructors); of the reference's nodes in this header only dR_Normalization
 * belongs to the CNN layer path served here. */
#ifndef DR_NODES_MISC_FWD_H
#define DR_NODES_MISC_FWD_H
#include "deepRACIN.h"
#endif
