// Prefill attention with a bias by distance and a query temperature: the kernel of attn_prefill.hip,
// compiled with these extras (see there), for head sizes up to 128.  Entry point: da_attn_prefill_rel.
#define PF_REL 1
#include "attn_prefill.hip"
