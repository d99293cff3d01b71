// Which keys a query may read beside the causal rule j <= p.  This header is the one place
// where a rule is defined: the cache manager (which pages a request still needs) and every
// attention kernel (which keys a query scores) take the rule from here, and the Python side
// reads the names, in the order of their codes, from either library.
//
// A rule is "the query at position p reads the keys first_visible(p) .. p".  A new rule is a
// new code, its name, and its case in sp_first_visible.
//
// The includer defines SP_VIS_FN (the function qualifiers of its compiler) before including.
#pragma once

enum { SP_VIS_FULL = 0, SP_VIS_CHUNK = 1, SP_VIS_WINDOW = 2, SP_VIS_COUNT = 3 };
#define SP_VIS_NAMES "full,chunk,window"

// Whether the rule uses its size (`span`), which must then be at least 1.
SP_VIS_FN bool sp_vis_has_span(int vis) { return vis != SP_VIS_FULL; }

// The most positions before its own that a query may read (-1: no bound): what the cache
// manager sizes a group's pool by.
SP_VIS_FN long sp_vis_lookback(int vis, int span) { return sp_vis_has_span(vis) ? (long)span - 1 : -1; }

// First position that a query at position p may read (the last is p itself).
template <typename I>
SP_VIS_FN I sp_first_visible(I p, int vis, int span) {
    if (vis == SP_VIS_CHUNK) return (p / span) * span;
    if (vis == SP_VIS_WINDOW) return p - span + 1 > 0 ? p - span + 1 : 0;
    return 0;
}
