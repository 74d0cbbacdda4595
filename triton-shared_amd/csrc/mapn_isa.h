// Instruction set of the fused-map interpreter kernel: shared by the planner, which assembles the
// register program, and the kernel, which runs it.  Plain C++, no device code.
#pragma once
#include <cstdint>

namespace tts {

enum MapOp : uint8_t {
  MO_MOV, MO_ADD, MO_SUB, MO_MUL, MO_DIV, MO_MAXNUM, MO_MINNUM, MO_MAXIMUM, MO_MINIMUM, MO_NEG, MO_ABS,
  MO_EXP, MO_EXP2, MO_LOG, MO_LOG2, MO_SQRT, MO_RSQRT, MO_SIN, MO_COS, MO_TANH, MO_ERF, MO_FLOOR, MO_CEIL, MO_FMA,
  MO_SELECT, MO_AND, MO_OR, MO_XOR,
  MO_CMP_OEQ, MO_CMP_ONE, MO_CMP_OLT, MO_CMP_OLE, MO_CMP_OGT, MO_CMP_OGE, MO_CMP_UNE, MO_CMP_UEQ, MO_CMP_ULT, MO_CMP_ULE,
  MO_CMP_UGT, MO_CMP_UGE, MO_CMP_ORD, MO_CMP_UNO,
};
constexpr int MAPN_MAX_IN = 6, MAPN_MAX_OUT = 2, MAPN_MAX_INS = 48, MAPN_MAX_IMM = 24, MAPN_MAX_REGS = 12;
// An operand is a register, the result of the instruction before (kept in hardware registers, so
// chains of ops do not go through the register file), or an immediate.
enum MapSrc : uint8_t { MS_REG = 0, MS_PREV = 1, MS_IMM = 2 };
struct MapIns {
  uint8_t op, dst, a, b;   // a, b, c: register number or immediate index, by the operand's kind
  uint8_t c;
  uint8_t kinds;           // MapSrc of a | b << 2 | c << 4; bit 6: the result is not written to the register file
  uint8_t round;           // 0: fp32 result, 1: round to fp16, 2: round to bf16
  uint8_t pad;
};
static_assert(sizeof(MapIns) == 8, "two 32-bit words per instruction");

}  // namespace tts
