// Declares the named Init / Exec globals of every native tile configuration, one pair per line
// of the generated lists in aq_bmma_impl/ (the role of the reference's
// engine/mma_any/aq_bmma_library.h and aq_bmma_impl/aq_bmma_w*.h).  As there, a combination is
// compiled in when its W{p}A{q} macro is defined; define ABQ_ALL_COMBOS for all twelve.
#pragma once
#include "mma_any/aq_bmma_op.h"

#ifdef ABQ_ALL_COMBOS
#define W2A2
#define W2A4
#define W2A6
#define W2A8
#define W3A3
#define W3A8
#define W4A4
#define W4A8
#define W5A5
#define W6A6
#define W7A7
#define W8A8
#endif

#ifndef AQ_CONFIG
#define AQ_CONFIG(...) AQ_DECL_FUN(AqBMMA, __VA_ARGS__)
#define AQ_CONFIG_DEFINED_BY_LIBRARY_H
#endif

#ifdef W2A2
#include "mma_any/aq_bmma_impl/aq_bmma_w2a2.inc"
#endif
#ifdef W2A4
#include "mma_any/aq_bmma_impl/aq_bmma_w2a4.inc"
#endif
#ifdef W2A6
#include "mma_any/aq_bmma_impl/aq_bmma_w2a6.inc"
#endif
#ifdef W2A8
#include "mma_any/aq_bmma_impl/aq_bmma_w2a8.inc"
#endif
#ifdef W3A3
#include "mma_any/aq_bmma_impl/aq_bmma_w3a3.inc"
#endif
#ifdef W3A8
#include "mma_any/aq_bmma_impl/aq_bmma_w3a8.inc"
#endif
#ifdef W4A4
#include "mma_any/aq_bmma_impl/aq_bmma_w4a4.inc"
#endif
#ifdef W4A8
#include "mma_any/aq_bmma_impl/aq_bmma_w4a8.inc"
#endif
#ifdef W5A5
#include "mma_any/aq_bmma_impl/aq_bmma_w5a5.inc"
#endif
#ifdef W6A6
#include "mma_any/aq_bmma_impl/aq_bmma_w6a6.inc"
#endif
#ifdef W7A7
#include "mma_any/aq_bmma_impl/aq_bmma_w7a7.inc"
#endif
#ifdef W8A8
#include "mma_any/aq_bmma_impl/aq_bmma_w8a8.inc"
#endif

#ifdef AQ_CONFIG_DEFINED_BY_LIBRARY_H
#undef AQ_CONFIG
#undef AQ_CONFIG_DEFINED_BY_LIBRARY_H
#endif
