// Bit-level definition of the streaming KV format consumed by the fused decode kernel.
//
// Token order of a unit (one KV head of one layer): class 0 = 2-bit V tokens, class 1 = 4-bit,
// class 2 = 8-bit, class 3 = fp16 V (zone B); inside a class the packer's order is kept, so
// token t of a class is row t of that class in the padded source tensors.  Every class is
// padded to whole tiles of 64 tokens; pad tokens carry zero bytes and are masked in the kernel.
//
// "Operand" = the four fp16 values one lane feeds to v_mfma_f32_4x4x4_16b_f16.  Packed fields
// are extracted two at a time with one shift+mask: a dword with fields of width w has
// nf = 32/w fields; pair i = (field i, field i + nf/2); operand s = (pair 2s, pair 2s+1), i.e.
//     operand s, element k  <->  field 2*s + (k >> 1) + (k & 1) * nf/2.
// The raw field value v is used as the fp16 bit pattern (a subnormal equal to v * 2^-24); the
// matrix cores keep fp16 subnormals, and the 2^24 factor is folded into a power-of-two scale.
//
// K tile (64 tokens): every token has a row of R = d8 + d4 + d2 dwords: first d8 dwords of
// 8-bit fields, then d4 dwords of 4-bit fields, then d2 dwords of 2-bit fields.  Operand
// ("step") numbering runs through the row: an 8-bit dword is 1 step, a 4-bit dword 2, a
// 2-bit dword 4; slot = 4*step + k indexes the unit's slot table (RdkvSlot) which names the
// query channel and the channel's scale / zero-point.  Rows are stored in chunks of up to 4
// dwords, chunk c of token t at  tile + 1024*c + t*4*wc  with wc = min(4, R - 4c), so a
// wavefront (lane = token) reads each chunk with one fully coalesced load.
//
// V tile (64 tokens = 16 quads of 4 tokens): lane l owns channels l and l+64.  Element k of
// an operand is token 4*quad + k.  Lane dword i of a tile lives at
//     tile + ((i >> 2) * 64 + l) * 16 + (i & 3) * 4,
// so a lane loads 16 B at a time and a wavefront 1 KiB contiguous.  Per class:
//   8-bit : dword i = 2*quad + j        -> operand 0 is (quad, channel l + 64*j)       32 dwords
//   4-bit : dword i = quad              -> operand s is (quad, channel l + 64*s)       16 dwords
//   2-bit : dword i = quad >> 1         -> operand s is (2*i + (s >> 1), l + 64*(s&1))  8 dwords
//   fp16  : dwords 4*quad + 2*j + {0,1} -> the four fp16 values of (quad, l + 64*j)    64 dwords
//
// Per token of a quantized class: one dword {scale fp16 | zp fp16 << 16} at sz + 4*token.
#pragma once

#include <stdint.h>

#define RDKV_TILE 64
#define RDKV_MAX_STEPS 40  // (128 channel slots + up to 3 + 7 + 15 pad slots of the three widths) / 4

static __host__ __device__ inline int rdkv_field_of(int s, int k, int nf) {
  return 2 * s + (k >> 1) + (k & 1) * (nf >> 1);
}
// inverse: field f of a dword with nf fields -> operand s and element k
static __host__ __device__ inline void rdkv_operand_of(int f, int nf, int *s, int *k) {
  const int half = nf >> 1;
  const int hi = f >= half;
  const int r = f - hi * half;
  *s = r >> 1;
  *k = ((r & 1) << 1) | hi;
}

static __host__ __device__ inline int rdkv_v_tile_bytes(int cls) { return 2048 << cls; }
