// Decode attention with a bias by distance and a query temperature: the kernel of attn_decode.hip,
// compiled with these extras (see there).  Entry point: da_attn_decode_rel.
#define DEC_REL 1
#include "attn_decode.hip"
