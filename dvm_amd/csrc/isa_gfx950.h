// Tile bytecode for the gfx950 device VM. Shared by the host emitter and the
// HIP interpreter kernels, so it is plain C structs and enums only.
//
// This plays the role the reference's src/isa.h plays for its targets
// (instruction ids src/isa.h:59-228, entry word src/isa.h:2388-2448), but the
// unit of interpretation is different: values live in per-lane registers, an
// instruction works on E consecutive elements per lane, and operands are
// addressed through stride descriptors instead of tile buffers in local
// memory.
#ifndef DVM_ISA_GFX950_H_
#define DVM_ISA_GFX950_H_

#include <stdint.h>

#define DVM_PARAM_BYTES 4096          // program blob travels as a kernel argument
#define DVM_PARAM_WORDS (DVM_PARAM_BYTES / 8)
#define DVM_VEC_E 8                   // consecutive elements per lane per slab (one or two 128-bit accesses)
// Slabs per lane per instruction. The vector VM is built twice: with 2 (kernels dvm_vm_vec_*: up to 1024
// lanes per workgroup) and with 4 (dvm_vm_vec_*_u4: half the instruction dispatches per element, more
// registers per lane, up to 512 lanes per workgroup); VS_WIDE in the header's schedule word selects the latter.
#ifndef DVM_VEC_U
#define DVM_VEC_U 2
#endif
#define DVM_VEC_U_WIDE 4
#define DVM_VEC_NREG 16               // V register slots per lane (local memory, sized per program)
#define DVM_VEC_NSREG 8               // one-float S registers per lane (VGPRs)
#define DVM_VEC_NSLOT 2               // concurrent reduce accumulators per sweep
#define DVM_VEC_MAXR 4                // max kept dims and max reduced dims after merging
#define DVM_VEC_MAXMEM 24             // memory operand descriptors per program

// ---- entry types ---------------------------------------------------------
enum {
  VE_VECTOR = 1,  // pointwise / broadcast / reduce program (vm_vector)
  VE_CUBE = 2,    // MFMA matmul tile loop + interpreted epilogue (vm_cube)
  VE_ATTN = 3,    // two MFMA stages with online softmax between them (vm_attn)
};

// ---- element types of memory operands ------------------------------------
enum {
  VDT_BOOL = 0,  // uint8 0/1 in memory, 0.0f/1.0f in registers
  VDT_F16 = 1,
  VDT_BF16 = 2,
  VDT_F32 = 3,
  VDT_I32 = 4,
  // No memory behind it: the element at offset i of the operand is the int32 value addr + i. With stride 1 along one
  // axis and 0 along the others it is that axis's coordinate (the position a one-hot compares its indices with).
  // Loads only, never with VMF_ALIGNED (the 128-bit paths would read memory).
  VDT_IOTA = 5,
};

// ---- schedules -------------------------------------------------------------
enum {
  VS_POINTWISE = 0,  // lanes enumerate the whole (kept) index space, no reduce
  VS_REDX = 1,       // innermost axis is reduced: a team of lanes strides the reduce space of one output
  VS_REDY = 2,       // innermost axis is kept: lanes own output groups, wave rows partition the reduce space
  VS_KIND_MASK = 0xf,
  VS_WIDE = 0x10,    // flag: the program is laid out for DVM_VEC_U_WIDE slabs per lane (the *_u4 kernels)
  // flag (VS_REDX only): every sweep is a load of a contiguous operand followed by at most DVM_VEC_SWEEP_BODY
  // instructions out of: float binaries (add .. max) on immediates, S registers, the accumulator or memory operands
  // that walk the reduced index space like the load (or not at all), float unaries, roundings, float reduces, stores,
  // loads of further operands that walk like the first;
  // between the sweeps nothing touches a V register; the kept and the reduced index space have at most two axes
  // each. Such a program may run on the sweep build of the VM
  // (dvm_vm_vec_rx_sw), which decodes a sweep's body once per sweep instead of once per instruction and round; the
  // generic kernel runs it as well and gives the same bits.
  VS_SWEEPS = 0x20,
};
#define DVM_VEC_SWEEP_BODY 6
// Local memory at the start of a vector program's segment, in doubles: what the lanes of a workgroup combine their
// reduce partials through. One double per lane; eight (one per element of a lane's group) on the schedule that keeps
// the innermost axis. The V registers lie behind it.
#define DVM_VEC_RED_SCRATCH_DOUBLES(sched, threads) ((((sched) & 0xfu) == 2u ? 8u : 1u) * (threads))

// ---- opcodes ---------------------------------------------------------------
// The interpreter is an accumulator machine. Per lane, `acc` holds U slabs of E
// elements (U*E values); one instruction transforms all of them. Opcodes below
// VOP_SRC_BASE take no source operand, the others fetch one (kind field).
enum {
  VOP_END = 0,
  VOP_LDR = 1,       // acc = vreg[a]
  VOP_LDS = 2,       // acc = splat(sreg[a])
  VOP_LDI = 3,       // acc = splat(imm)
  VOP_STR = 4,       // vreg[a] = acc           (sub: VF_F32 two slots, VF_16 one slot of packed halves)
  VOP_STS = 5,       // sreg[a] = acc[0][0]
  VOP_ST = 6,        // mem[a] = acc
  VOP_UN = 7,        // acc = f(acc), sub = VU_*
  VOP_CAST = 8,      // container conversion, sub = VC_*
  VOP_RED = 9,       // slot[a] (sub = VR_*) accumulates acc      (inside a sweep)
  VOP_SWEEP = 10,    // start of a loop over the reduce index space; imm = slot kinds, 4 bits each
  VOP_ENDSWEEP = 11, // next round, or fall through and combine the slots across lanes
  VOP_FIN = 12,      // acc = combined slot[a]
  VOP_UNI_BEGIN = 13,// start of a run whose values are the same in every lane of a team; imm = distance in
                     // instructions to the matching VOP_UNI_END. When the team is the whole workgroup only its
                     // first wave executes the run, the others jump to the end
  VOP_UNI_END = 14,  // end of the run: the first wave's S registers and accumulator value are handed to the
                     // other waves through local memory
  VOP_SRC_BASE = 16,
  VOP_LD = 16,       // acc = mem[a]             (kind is always VK_MEM)
  VOP_BINF = 17,     // acc = acc (sub = VB_*) src, float class
  VOP_BINI = 18,     // acc = acc (sub = VBI_*) src, int32 class
  VOP_CMP = 19,      // acc = acc (sub = VCMP_*, +8 for int32) src ? 1 : 0 in the operand's container
  VOP_MSK = 20,      // mask = src != 0          (per element predicate)
  VOP_MOVM = 21,     // acc = mask ? src : acc
  VOP_LDX = 22,      // acc = mem[a] at the operand's offsets plus acc (int32, in elements): a gather. kind is VK_MEM
};

// source kinds (bits 16..19). VK_SREG2 (VOP_BINF only) chains two float binaries with S-register operands in
// one instruction: acc = (acc (sub) sreg[a]) (sub2) sreg[a2], each result rounded by its own rnd field; the
// second operation sits in the immediate: [7:0] sub2, [15:8] a2, [17:16] rnd2.
enum { VK_REG = 0, VK_IMM = 1, VK_MEM = 2, VK_ACC = 3, VK_SREG = 4, VK_SREG2 = 5 };
// result rounding (bits 20..21): value is rounded to that format and widened back
enum { VRND_NONE = 0, VRND_F16 = 1, VRND_BF16 = 2 };
// V register storage formats
enum { VF_F32 = 0, VF_F16 = 1, VF_BF16 = 2 };

// float binary sub-ops (R* = operands reversed: src op acc)
enum {
  VB_ADD = 0, VB_SUB, VB_RSUB, VB_MUL, VB_DIV, VB_RDIV, VB_MIN, VB_MAX, VB_AND, VB_OR, VB_POW, VB_RPOW,
  VB_DIV_APPROX, VB_RDIV_APPROX,  // matmul epilogues only: acc * rcp(src), src * rcp(acc) with v_rcp_f32
};
// int32 binary sub-ops
// VBI_WRAP: an index into an axis of extent src: acc + src where acc is negative, then clipped to [0, src - 1]
enum { VBI_ADD = 0, VBI_SUB, VBI_RSUB, VBI_MUL, VBI_MIN, VBI_MAX, VBI_WRAP };
// unary sub-ops
enum {
  VU_SQRT = 0, VU_ABS, VU_LOG, VU_EXP, VU_ISFINITE, VU_ROUND, VU_FLOOR, VU_CEIL, VU_TRUNC, VU_IABS,
  // matmul epilogues only. VU_EXP_SCALED: acc = exp(acc * imm), the product rounded to fp32 first (the fused form
  // of a multiply by a constant followed by Exp). The _APPROX forms use the hardware approximations (v_exp_f32,
  // v_log_f32, v_sqrt_f32: one ulp of fp32); the host picks them under VCF_APPROX_MATH.
  VU_EXP_SCALED, VU_EXP_APPROX, VU_EXP_SCALED_APPROX, VU_LOG_APPROX, VU_SQRT_APPROX,
  // matmul epilogues under VCF_APPROX_MATH only: the four (three) instructions of x / (exp(x * imm) + 1) and of
  // 1 / (exp(x * imm) + 1) in one dispatch, every intermediate rounded to fp32 as the separate instructions do
  // (SiLU and the logistic function with imm = -1); the host joins them when none of the four rounds to a 16-bit type
  VU_SILU_APPROX, VU_SIGMOID_APPROX,
};
// compare sub-ops (same order as dvm::BinaryType kEqual..kLessEqual); +VCMP_INT for int32 operands
enum { VCMP_EQ = 0, VCMP_NE, VCMP_GT, VCMP_GE, VCMP_LT, VCMP_LE, VCMP_INT = 8 };
// cast kinds
enum {
  VC_F2I = 0,    // float container -> int32 (C truncation)
  VC_I2F = 1,    // int32 -> float (then optional rounding via rnd field)
  VC_RND = 2,    // float -> float rounded per rnd field (f32->f16, f32->bf16)
  VC_F2B = 3,    // float -> bool container (x != 0 ? 1.0 : 0.0)
};
// reduce kinds (low 4 bits of VOP_RED's sub field), and two modifiers of VOP_RED
enum { VR_SUM = 0, VR_MAX = 1, VR_MIN = 2, VR_NONE = 15 };
#define VRF_SQUARE 0x10u  // acc = acc * acc (the fp32 product) first; the multiply of a sum of squares rides in the reduce
#define VRF_PAIR 0x40u    // VOP_RED into slot 0: the same value, squared, also goes to slot 1 (sum and sum of squares in one instruction)
#define VRF_INT 0x20u     // VOP_RED (max / min) and VOP_FIN: the values are int32 bit patterns, compared as integers

// instruction word:
//   [6:0] opcode  [7] VI_ENDS  [15:8] sub  [19:16] src kind  [21:20] rnd  [22] VI_UNIFORM  [23] VI_SAME_OFFS
//   [31:24] a (register / memory operand / slot index)   [63:32] imm32
// VI_UNIFORM (vector VM, arithmetic without a memory or V-register operand): every element of the lane's
// accumulator holds the same value, the instruction may compute one and copy it.
// VI_SAME_OFFS (vector VM, memory instructions): the operand has the strides of the previous memory
// instruction of the same round, whose element offsets are reused.
// Re-reading less in the second sweep over a tensor (vector VM, schedule that reduces the innermost axis):
//  VI_LD_KEEP_WR / VI_LD_KEEP_RD (VOP_LD that opens a sweep; the rnd field is free there; imm[15:0] = number of
//    rounds): the first load parks the slabs of its first rounds in local memory, the load that opens a later
//    sweep over the same operand takes those rounds from there instead of from memory. imm[17:16] = p (0 or 1):
//    what is parked is the accumulator behind the p instructions that follow the load, which both sweeps have in
//    common (x + residual), and the reading sweep skips those p instructions in a parked round, so their memory
//    operands are not read again either. imm[21:20] = VF_*: how the value is parked (fp32: two 16-byte planes per
//    slab; fp16 / bf16, when the last common instruction rounds to that type: one);
//  VSW_REVERSE (sub field of VOP_SWEEP): the sweep walks its rounds last to first, so that it starts with
//    what the sweep before it read last (still in the L2 cache) and ends with the parked rounds.
#define VI_LD_KEEP_WR (1u << 20)
#define VI_LD_KEEP_RD (1u << 21)
#define VSW_REVERSE 1u
// VI_LD_PAIR (lowest bit of VOP_LD's sub field, vector VM): the next instruction is a VOP_BINF whose operand is a
// memory operand with VI_SAME_OFFS. The load may fetch both operands at once (one trip to memory for the pair)
// and finish the binary in the same dispatch; an interpreter that ignores the flag computes the same.
#define VI_LD_PAIR (1u << 8)
// VI_LD_RED2 (second bit of VOP_LD's sub field; schedule that reduces the innermost axis): the body of the sweep
// is this load and one float VOP_RED with VI_ENDS behind it (a statistics sweep). The load may fetch this round
// and the next in one trip to memory, do the reduce for both and step two rounds; an interpreter that ignores
// the flag computes the same, round by round. (The partials of the two orders are the same sums: the reduce
// accumulates per lane in the order of the rounds either way.)
#define VI_LD_RED2 (1u << 9)
// VI_ENDS (top bit of the opcode byte; set on every VOP_ENDSWEEP, and on a store or reduce that took over the
// VOP_ENDSWEEP behind it): the instruction closes the round of its sweep. One bit, so that the decoder finds the
// next pc without comparing opcodes.
#define VI_ENDS 0x80u
#define VI_UNIFORM (1u << 22)
#define VI_SAME_OFFS (1u << 23)
// VI_OFFS_ASIDE (top bit of the sub field; vector VM, a VOP_BINF / VOP_BINI / VOP_CMP / VOP_MSK / VOP_MOVM with a memory
// operand): the operand walks memory differently from the memory instruction before it, and its offsets are not
// what a later VI_SAME_OFFS refers to: that still means the instruction before this one (x * w stored where x came
// from: the store reuses the load's offsets although the weight row was read in between).
#define VI_OFFS_ASIDE (1u << 15)
// VI_PRE_SREG (top bit of the immediate of a VOP_BINF with a memory operand, whose immediate is otherwise unused): an
// S-register float binary runs in front of it, acc = acc (sub2) sreg[a2], rounded by rnd2, in the same dispatch (the
// memory operand is on its way meanwhile): imm[7:0] sub2 (VB_ADD, VB_SUB, VB_RSUB or VB_MUL), imm[15:8] a2,
// imm[17:16] rnd2. x * rstd * w of a normalisation is one instruction instead of two.
#define VI_PRE_SREG (1u << 31)
#define VI_MAKE(op, sub, kind, rnd, a, imm)                                                     \
  ((uint64_t)(op) | ((uint64_t)(sub) << 8) | ((uint64_t)(kind) << 16) | ((uint64_t)(rnd) << 20) | \
   ((uint64_t)(a) << 24) | ((uint64_t)(uint32_t)(imm) << 32))
#define VI_OP(w) ((uint32_t)(w) & 0x7fu)
#define VI_SUB(w) (((uint32_t)(w) >> 8) & 0xffu)
#define VI_KIND(w) (((uint32_t)(w) >> 16) & 0xfu)
#define VI_RND(w) (((uint32_t)(w) >> 20) & 0x3u)
#define VI_A(w) (((uint32_t)(w) >> 24) & 0xffu)
#define VI_IMM(w) ((uint32_t)((w) >> 32))

// One axis of an index space, with the constants of a multiply-shift division
// (q = (mulhi(n, magic) + n) >> shift, valid for n < 2^31).
typedef struct {
  uint32_t extent;  // for the innermost domain axis: number of E-groups
  uint32_t magic;
  uint32_t shift;
  uint32_t pad;
} VDim;

// A memory operand: base address plus element strides against the kept list
// and the reduced list (position 0 = fastest varying). The stride of the
// innermost domain axis is 0 (operand broadcast along it: one element is
// loaded and replicated), 1 (E consecutive elements) or, with VMF_GATHER, any.
typedef struct {
  uint64_t addr;
  uint32_t dtype;                  // VDT_*
  uint32_t flags;                  // VMF_*
  uint32_t kstride[DVM_VEC_MAXR];
  uint32_t rstride[DVM_VEC_MAXR];
} VMemDesc;
// VMF_GATHER: the innermost stride is neither 0 nor 1 (a transposing or element-skipping view); it sits in
// flags[31:8] and in the stride entry of the innermost axis, and the operand is accessed element by element.
enum { VMF_VEC = 1 /* innermost stride 1 */, VMF_ALIGNED = 2 /* every E-group starts 16-byte aligned */, VMF_GATHER = 4 };

typedef struct {
  uint32_t entry;        // VE_VECTOR
  uint32_t sched;        // VS_* | VS_WIDE
  uint32_t n_mem;
  uint32_t n_code;       // instruction words
  uint32_t n_kdim;
  uint32_t n_rdim;
  uint32_t team_log2;    // REDX: lanes per team; REDY: lanes along the kept space (tx)
  uint32_t team_is_block;// REDX: team spans the whole workgroup
  uint32_t n_kidx;       // size of the kept index space (groups if the innermost axis is kept)
  uint32_t n_ridx;       // size of the reduced index space (groups if the innermost axis is reduced)
  uint32_t inner_extent; // elements along the innermost domain axis
  uint32_t inner_reduced;// innermost axis belongs to the reduced list
  uint32_t n_items;      // work items (grid-strided over workgroups)
  uint32_t mem_off;      // word offset of VMemDesc[n_mem]
  uint32_t code_off;     // word offset of the instruction words
  uint32_t n_vslot;      // V register slots in use (each U*16 bytes per lane of local memory)
  // A reduce shared between workgroups (both 0 otherwise): the outermost kept axis numbers the parts of the reduced
  // index space, r_chunk indices each (whole rounds; the last part may be short or empty); coordinate c of a lane along
  // that axis is kidx / k_per_chunk, and the lane reduces the indices [c * r_chunk, min(n_ridx, (c + 1) * r_chunk)).
  uint32_t r_chunk;
  uint32_t k_per_chunk;
  uint32_t pad[2];       // (keeps the axis tables 16-byte aligned: the interpreter reads them as 128-bit words)
  VDim kdims[DVM_VEC_MAXR];
  VDim rdims[DVM_VEC_MAXR];
} VVecHeader;            // 80 + 128 = 208 bytes

// ---- matmul programs (VE_CUBE) ---------------------------------------------------
// C[b][m][n] = sum_k A[b][m][k] * B[b][k][n], fp32 accumulation on MFMA, then an epilogue program
// in the vector VM's instruction words runs on every accumulator fragment (acc = the 16 values a
// lane holds of one 32x32 tile) before anything is stored: VOP_CAST / VOP_UN / VOP_BINF / VOP_BINI /
// VOP_CMP / VOP_MSK / VOP_MOVM with VK_IMM, VK_ACC, VK_MEM (stride-addressed, so a bias row is a
// stride-0 operand) or VK_REG (DVM_CUBE_NTEMP temporaries), VOP_STR / VOP_LDR on those
// temporaries, VOP_ST to one or more outputs.
#define DVM_CUBE_MAXMEM 12
#define DVM_CUBE_NTEMP 4

typedef struct {
  uint64_t addr;
  uint32_t dtype;     // VDT_*
  uint32_t flags;
  uint32_t stride_n;  // element strides against the output's n, m and the two batch axes (0 = broadcast)
  uint32_t stride_m;
  uint32_t stride_b0;
  uint32_t stride_b1;
} VCubeMem;

typedef struct {
  uint32_t entry;      // VE_CUBE
  uint32_t dtype;      // VDT_F16 or VDT_BF16 (operand type; accumulation is fp32)
  uint32_t m, n, k;
  uint32_t trans_a;    // A is stored [k][m]
  uint32_t trans_b;    // B is stored [n][k]
  uint32_t lda, ldb;   // leading dimensions in elements
  uint32_t nb0, nb1;   // batch extents (outer, inner); 1 when absent
  uint32_t a_sb0, a_sb1, b_sb0, b_sb1;  // batch strides in elements (0 = broadcast)
  uint32_t tile;       // block tile: 0 = 256x256, 1 = 128x128, 2 = 64x64 (four waves), 3 = 256x256 on eight waves (512 lanes)
  uint32_t tiles_m, tiles_n;
  uint32_t n_mem, n_code;
  uint32_t mem_off, code_off;  // word offsets
  uint32_t fast;       // k is a multiple of 64 and every 8-element operand chunk is 16-byte aligned: full tiles take the vector path
  uint32_t epi_flags;  // VCF_*
  uint64_t a_addr, b_addr;
  uint32_t k_split;    // VCF_SPLITK_*: parts the k axis is cut into (>= 2), each k_chunk long (a multiple of 64; the last
  uint32_t k_chunk;    // may be shorter), and the fp32 partial tiles: [k_split][tiles][tile vectors][lanes] of 16 bytes
  uint64_t part_addr;
  // Grouped products (VCG_*; nb0 = 1, nb1 = the number of groups): a list of nb1 int64 (group_i32: int32) values in
  // device memory, the upper bounds of the groups' ranges (VCG_*_BOUND: ascending) or their sizes (VCG_*_SIZE), read
  // by the kernel when it starts. VCG_M_*: group g owns the rows [bound[g-1], bound[g]) of A and of the output and
  // multiplies them with matrix g of B; the output has no batch axis, and a tile that crosses a bound is computed
  // once per group that owns rows of it, each storing only its rows. VCG_K_*: group g multiplies the columns
  // [bound[g-1], bound[g]) of A with the same rows of B into matrix g of the output (zeros for an empty range).
  uint64_t group_addr;
  uint32_t group_mode;
  uint32_t group_i32;
} VCubeHeader;
enum { VCG_NONE = 0, VCG_M_BOUND = 1, VCG_M_SIZE = 2, VCG_K_BOUND = 3, VCG_K_SIZE = 4 };
#define DVM_CUBE_MAX_GROUPS 2048u

// VCubeHeader::epi_flags
// Every store of the epilogue writes fp16 or bf16 and the program holds only operators that are continuous in
// their inputs (no compare, select, rounding to integers, conversion to int32): the host has replaced exp, log,
// sqrt and division by their _APPROX forms (one ulp of fp32; the 16-bit rounding is four orders coarser).
#define VCF_APPROX_MATH 1u
// Split k, for products with fewer tiles than compute units and a long k axis: two launches of the same program.
// VCF_SPLITK_PARTIAL: tiles * k_split workgroups; each multiplies one part of the k axis and writes its accumulators
// to part_addr as the lanes hold them, no epilogue. VCF_SPLITK_COMBINE: one workgroup per tile adds the k_split
// partials in ascending k order (fp32, the same order on every run) and runs the epilogue on the sum.
// The epilogue is [add of a memory operand (a bias row)] [rounding to a float type] store: the kernel does it in
// place, without walking the program through the interpreter (a dispatch costs more than this whole epilogue).
#define VCF_PLAIN_STORE 8u
// The epilogue holds only loads, stores, rounding, the temporary 0, float binaries (add, sub, rsub, mul, div, rdiv
// and their hardware forms, min, max) and the unaries abs and the hardware's exp / scaled exp / log / sqrt: it runs
// through a build of the interpreter's pass without the arms of everything else, which needs half the registers
// (what calling the pass costs is the registers it saves).
#define VCF_SLIM 16u
// The program starts with [add of a bias row: one value per column, the same for every row] [rounding to the
// operand type] (or, in place of the rounding, consists of nothing but one store of the operand type behind the
// add), which is what every product's program starts with unless its bias walks memory some other way.
// The kernel then does these two in the layout the accumulators have (a lane's column is fixed there: one bias value
// per fragment), hands the epilogue the whole tile as 16-bit values in one pass, and the interpreter starts behind
// them. (As fp32 only half a 256 x 256 tile fits local memory, and the second half's accumulators stayed live across
// the first half's pass: registers saved to scratch memory around the call.)
#define VCF_DUMP16 32u
#define VCF_SPLITK_PARTIAL 2u
#define VCF_SPLITK_COMBINE 4u

// Dynamic local memory a VE_CUBE launch needs for block tile `bt` (256, 128 or 64): the operand tiles of the k
// loop (two buffers of 64 k per operand; for the 256 tile the same bytes as four stage buffers of 32 k), or what
// the epilogue reads back: half the tile as fp32 accumulators, or the whole tile as 16-bit values (VCF_DUMP16).
#define DVM_CUBE_LDS_LOOP_BYTES(bt) (2u * (2u * (bt)) * 64u * 2u)
#define DVM_CUBE_LDS_DUMP32_BYTES(bt) (((bt) >= 128u ? (bt) / 2u : (bt)) * ((bt) + 4u) * 4u)
#define DVM_CUBE_LDS_DUMP16_BYTES(bt) ((bt) * ((bt) + 8u) * 2u)
#define DVM_CUBE_MAX2(a, b) ((a) > (b) ? (a) : (b))
#define DVM_CUBE_LDS_BYTES(bt) \
  DVM_CUBE_MAX2(DVM_CUBE_LDS_LOOP_BYTES(bt), DVM_CUBE_MAX2(DVM_CUBE_LDS_DUMP32_BYTES(bt), DVM_CUBE_LDS_DUMP16_BYTES(bt)))
// (a grouped product keeps its tables behind that: 8 bytes per group)

// ---- fused attention programs (VE_ATTN) -------------------------------------------
// O[b] = softmax(Q[b] K[b]^T * scale) V[b] for nb independent (batch, head) pairs, all operands row
// major with the head dimension contiguous: Q [nb][sq][d], K [nb][skv][d], V [nb][skv][d], O [nb][sq][d].
// One workgroup owns DVM_ATTN_BQ query rows and walks the keys in blocks of DVM_ATTN_BKV with an
// online softmax (running row max and sum), so the [sq][skv] score matrix never exists in memory.
#define DVM_ATTN_BQ 256
#define DVM_ATTN_BKV 64
#define DVM_ATTN_D 128                  // head dimension: this, or half of it
#define DVM_ATTN_D_OK(d) ((d) == DVM_ATTN_D || (d) == DVM_ATTN_D / 2)
#define DVM_ATTN_LDS_BYTES_D(d) (2u * 2u * DVM_ATTN_BKV * (d) * 2u)  // two buffers of a K block and a V block
#define DVM_ATTN_LDS_BYTES DVM_ATTN_LDS_BYTES_D(DVM_ATTN_D)

typedef struct {
  uint32_t entry;   // VE_ATTN
  uint32_t dtype;   // VDT_F16 or VDT_BF16
  uint32_t nb;      // batch * heads
  uint32_t sq, skv; // query rows, keys (a last block of fewer than DVM_ATTN_BKV keys is masked)
  uint32_t d;       // head dimension: 128 or 64 (DVM_ATTN_D_OK)
  float scale;      // applied to Q K^T before the softmax; positive
  uint32_t q_blocks;  // ceil(sq / DVM_ATTN_BQ)
  uint64_t q_addr, k_addr, v_addr, o_addr;
  // How Q, K, V, O (in this order) lie in memory: element stride from one row (query or key) to the next, and from
  // one (batch, head) pair to the next along the outer and the inner of two batch axes; pair b has the indices
  // (b / nb_inner, b % nb_inner). Every stride is a multiple of 8 elements (16 bytes). A dense [nb][rows][d] tensor
  // has row = d, outer = rows * d with nb_inner = 1; the heads-first view of a [batch][seq][heads][d] tensor has
  // row = heads * d, outer = seq * heads * d, inner = d with nb_inner = heads.
  uint32_t nb_inner;
  uint32_t row_stride[4], outer_stride[4], inner_stride[4];
  uint32_t pad;
} VAttnHeader;

typedef struct {
  uint64_t w[DVM_PARAM_WORDS];
} VmParam;

#endif  // DVM_ISA_GFX950_H_
