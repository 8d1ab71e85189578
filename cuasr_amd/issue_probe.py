"""Instruction-issue probe for gfx950: the measurements the hand-scheduled main loops
(csrc/gen_direct_asm.py) are designed around, and the ceiling they are judged against.

    python -m cuasr_amd.issue_probe --build      # writes and compiles cuasr_amd/lib/issue_probe (hipcc, no GPU needed)
    cuasr_amd/lib/issue_probe [iterations]       # runs it on the GPU, prints one line per loop

Every loop is one inline-asm block of the fp32 min-plus inner loop of an 8 x 8 register tile (64
groups of add, add, min3 = 128 terms per lane) or a variation of it, run by 256-thread workgroups,
1 to 4 per compute unit (= 1 to 4 waves per SIMD), with nothing else in the loop:
    add / min3 / min / fma / fmac alone   what one instruction kind issues at
    mix                                   the min-plus group itself: the ceiling of any min-plus kernel
    mix + SGPR operand                    a fragment broadcast through scalar registers
    mix + N LDS reads (4 / 8 / 16 bytes)  what fetching the fragments costs (results not consumed)
    mix + N waits / nops / scalar adds    what an instruction that does no arithmetic costs
    packed fp16 add / min / minimum3 / mix the same for two fp16 terms per instruction
    SDWA byte add / min3_i32 / mix         int8 operands widened by the add's own byte selects
    packed int16 multiply / min / mix      int8 operands as 16-bit integers (products fit): min-times, max-times
    fp64 add / max / mix (+ the same)     the same questions for 8-byte elements
Times are HIP events around the second of two launches; the clock is read inside the kernel
(shader cycle counter against the 100 MHz wall clock), so cycle figures are per measured clock.

    cuasr_amd/lib/issue_probe mfma               # the matrix instructions of the narrow element types instead

runs, for two seconds each and twice over, loops of nothing but v_mfma_i32_32x32x32_i8 / 16x16x64_i8 and
v_mfma_f32_32x32x16_f16 / 16x16x32_f16 (one wave per SIMD, 256 accumulator registers, eight A and eight B
fragments of random register contents) and prints rate and board power (hwmon power1_input) over the second
second: what the chip delivers through each shape on toggling operands at its power cap, which is what
csrc/mfma_direct_narrow.hip picks its instructions by.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "lib", "issue_probe")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

ACC = list(range(32, 96))
A0, A1 = list(range(96, 104)), list(range(104, 112))
B0, B1 = list(range(112, 120)), list(range(120, 128))
T = list(range(24, 32))


def mix(sgpr_b=False):
    groups, t = [], 0
    for i in range(8):
        for j in range(8):
            t0, t1 = T[t % 8], T[(t + 1) % 8]
            t += 2
            b0 = f"s{16 + j}" if sgpr_b else f"v{B0[j]}"
            b1 = f"s{24 + j}" if sgpr_b else f"v{B1[j]}"
            acc = ACC[i * 8 + j]
            groups.append([f"v_add_f32 v{t0}, {b0}, v{A0[i]}", f"v_add_f32 v{t1}, {b1}, v{A1[i]}",
                           f"v_min3_f32 v{acc}, v{acc}, v{t0}, v{t1}"])
    return groups


def mix_f16():
    """min-plus on packed fp16: acc[i][j] holds two columns; row i's fragment word holds two k (or two
    rows), picked by op_sel; 256 terms per lane in 192 instructions"""
    groups, t = [], 0
    for i in range(8):
        for j in range(8):
            t0, t1 = T[t % 8], T[(t + 1) % 8]
            t += 2
            acc = ACC[i * 8 + j]
            groups.append([f"v_pk_add_f16 v{t0}, v{A0[i]}, v{B0[j]} op_sel_hi:[0,1]",
                           f"v_pk_add_f16 v{t1}, v{A0[i]}, v{B1[j]} op_sel:[1,0] op_sel_hi:[1,1]",
                           f"v_pk_minimum3_f16 v{acc}, v{acc}, v{t0}, v{t1}"])
    return groups


def mix_i16():
    """min-times on int8 operands widened to packed int16 (a product of two int8 values is a 16-bit integer): two
    products and two minima per group of four terms -- there is no three-input packed integer minimum; 256 terms per
    lane in 256 instructions"""
    groups, t = [], 0
    for i in range(8):
        for j in range(8):
            t0, t1 = T[t % 8], T[(t + 1) % 8]
            t += 2
            acc = ACC[i * 8 + j]
            groups.append([f"v_pk_mul_lo_u16 v{t0}, v{A0[i]}, v{B0[j]} op_sel_hi:[0,1]",
                           f"v_pk_mul_lo_u16 v{t1}, v{A0[i]}, v{B1[j]} op_sel:[1,0] op_sel_hi:[1,1]",
                           f"v_pk_min_i16 v{acc}, v{acc}, v{t0}",
                           f"v_pk_min_i16 v{acc}, v{acc}, v{t1}"])
    return groups


def mix_i8():
    """min-plus on int8 operands with int32 accumulators: a register holds 4 k of one row (column); the add picks
    its bytes and widens them"""
    groups, t = [], 0
    for i in range(8):
        for j in range(8):
            t0, t1 = T[t % 8], T[(t + 1) % 8]
            t += 2
            acc = ACC[i * 8 + j]
            groups.append([f"v_add_u32_sdwa v{t0}, sext(v{A0[i]}), sext(v{B0[j]}) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_0 src1_sel:BYTE_0",
                           f"v_add_u32_sdwa v{t1}, sext(v{A0[i]}), sext(v{B0[j]}) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_1 src1_sel:BYTE_1",
                           f"v_min3_i32 v{acc}, v{acc}, v{t0}, v{t1}"])
    return groups


def sprinkle(groups, n, make):
    """n extra instructions spread evenly over the groups"""
    lines, every, c = [], (len(groups) // n if n else 10 ** 9), 0
    for gi, grp in enumerate(groups):
        if n and gi % every == 0 and c < n:
            lines.append(make(c))
            c += 1
        lines += grp
    return lines


def only(template, n=192):
    return [template.format(t=T[x % 8], acc=ACC[x % 64], a=A0[(x // 8) % 8], b=B0[x % 8], s=16 + x % 8) for x in range(n)]


def lds_read(width):
    regs = {32: list(range(4, 20)), 64: list(range(4, 20, 2)), 128: [4, 8, 12, 16]}[width]
    name = {32: lambda r: f"v{r}", 64: lambda r: f"v[{r}:{r + 1}]", 128: lambda r: f"v[{r}:{r + 3}]"}[width]
    return lambda c: f"ds_read_b{width} {name(regs[c % len(regs)])}, %0 offset:{(c * 1024) % 32768}"


def f64_mix():
    acc = [32 + 2 * i for i in range(32)]
    a = [96 + 2 * i for i in range(8)]
    b = [112 + 2 * i for i in range(4)]
    t = [16 + 2 * i for i in range(4)]
    r = lambda x: f"v[{x}:{x + 1}]"
    return [[f"v_add_f64 {r(t[(i * 4 + j) % 4])}, {r(a[i])}, {r(b[j])}",
             f"v_max_f64 {r(acc[i * 4 + j])}, {r(acc[i * 4 + j])}, {r(t[(i * 4 + j) % 4])}"] for i in range(8) for j in range(4)]


def kernels():
    k = {}  # name -> (lines, instructions counted, terms per lane, "f32" | "f64")
    flat = lambda g: [ln for grp in g for ln in grp]
    k["add_f32"] = (only("v_add_f32 v{t}, v{b}, v{a}"), 192, 0, "f32")
    k["add_f32_sgpr_operand"] = (only("v_add_f32 v{t}, s{s}, v{a}"), 192, 0, "f32")
    k["min3_f32"] = (only("v_min3_f32 v{acc}, v{acc}, v{b}, v{a}"), 192, 0, "f32")
    k["min_f32"] = (only("v_min_f32 v{acc}, v{acc}, v{b}"), 192, 0, "f32")
    k["fma_f32_vop3"] = (only("v_fma_f32 v{acc}, v{b}, v{a}, v{acc}"), 192, 0, "f32")
    k["fmac_f32_vop2"] = (only("v_fmac_f32 v{acc}, v{b}, v{a}"), 192, 0, "f32")
    k["bitop3_b32"] = (only("v_bitop3_b32 v{acc}, v{b}, v{a}, v{acc} bitop3:0x6a"), 192, 0, "f32")
    # packed fp16: two terms per instruction and lane; the fragment of one operand is broadcast by the
    # instruction's own half-word selects
    k["pk_add_f16"] = (only("v_pk_add_f16 v{t}, v{b}, v{a}"), 192, 0, "f32")
    k["pk_add_f16_broadcast"] = (only("v_pk_add_f16 v{t}, v{b}, v{a} op_sel:[1,0] op_sel_hi:[1,1]"), 192, 0, "f32")
    k["pk_min_f16"] = (only("v_pk_min_f16 v{acc}, v{acc}, v{b}"), 192, 0, "f32")
    k["pk_minimum3_f16"] = (only("v_pk_minimum3_f16 v{acc}, v{acc}, v{b}, v{a}"), 192, 0, "f32")
    k["pk_mul_f16"] = (only("v_pk_mul_f16 v{t}, v{b}, v{a}"), 192, 0, "f32")
    k["mix_f16"] = (flat(mix_f16()), 192, 256, "f32")
    for n in (6, 12):
        k[f"mix_f16_lds{n}_b128"] = (sprinkle(mix_f16(), n, lds_read(128)), 192, 256, "f32")
    # int8 operands, four to a register, widened by the add itself (SDWA byte selects with sign extension)
    k["add_u32_sdwa_bytes"] = (only("v_add_u32_sdwa v{t}, sext(v{b}), sext(v{a}) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_1 src1_sel:BYTE_2"), 192, 0, "f32")
    k["min3_i32"] = (only("v_min3_i32 v{acc}, v{acc}, v{b}, v{a}"), 192, 0, "f32")
    k["mix_i8_sdwa"] = (flat(mix_i8()), 192, 128, "f32")
    # int8 operands as packed int16 (min-times / max-times)
    k["pk_mul_lo_u16"] = (only("v_pk_mul_lo_u16 v{t}, v{b}, v{a}"), 192, 0, "f32")
    k["pk_min_i16"] = (only("v_pk_min_i16 v{acc}, v{acc}, v{b}"), 192, 0, "f32")
    k["mix_i16"] = (flat(mix_i16()), 256, 256, "f32")
    # an operand fetched from another lane of the quad by the add itself (a fragment shared by four lanes)
    k["add_f32_dpp_quad"] = (only("v_add_f32_dpp v{t}, v{b}, v{a} quad_perm:[1,1,1,1] row_mask:0xf bank_mask:0xf"), 192, 0, "f32")
    k["mix"] = (flat(mix()), 192, 128, "f32")
    k["mix_sgpr_b"] = (flat(mix(True)), 192, 128, "f32")
    for n in (4, 8, 16):
        for w in (64, 128):
            k[f"mix_lds{n}_b{w}"] = (sprinkle(mix(), n, lds_read(w)), 192, 128, "f32")
    for n in (16, 64):
        k[f"mix_waitcnt{n}"] = (sprinkle(mix(), n, lambda c: "s_waitcnt lgkmcnt(0)"), 192, 128, "f32")
        k[f"mix_nop{n}"] = (sprinkle(mix(), n, lambda c: "s_nop 0"), 192, 128, "f32")
        k[f"mix_salu{n}"] = (sprinkle(mix(), n, lambda c: "s_add_u32 s20, s20, 1"), 192, 128, "f32")
    g64 = f64_mix()
    k["add_f64"] = ([g[0] for g in g64] * 2, 64, 0, "f64")
    k["max_f64"] = ([g[1] for g in g64] * 2, 64, 0, "f64")
    k["mix_f64"] = (flat(g64), 64, 32, "f64")
    k["mix_f64_lds6_b128"] = (sprinkle(g64, 6, lds_read(128)), 64, 32, "f64")
    k["mix_f64_waitcnt8"] = (sprinkle(g64, 8, lambda c: "s_waitcnt lgkmcnt(0)"), 64, 32, "f64")
    k["mix_f64_nop32"] = (sprinkle(g64, 32, lambda c: "s_nop 0"), 64, 32, "f64")
    return k


MFMA_SECTION = r'''
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
__device__ unsigned mfma_rnd(unsigned x) { x ^= x << 13; x ^= x >> 17; x ^= x << 5; return x * 2654435761u; }
// KIND 0: i32_32x32x32_i8 (4 x 4 blocks), 1: i32_16x16x64_i8 (8 x 8), 2: f32_32x32x16_f16, 3: f32_16x16x32_f16
template <int KIND>
__global__ __launch_bounds__(256) void k_mfma(int *out, int iters) {
  unsigned s = mfma_rnd(threadIdx.x * 977u + blockIdx.x * 131071u + 12345u);
  v4i a[8], b[8];
  for (int i = 0; i < 8; ++i) for (int j = 0; j < 4; ++j) {
    s = mfma_rnd(s); unsigned x = s; s = mfma_rnd(s); unsigned y = s;
    if (KIND >= 2) { x = (x & 0x83ff83ffu) | 0x38003800u; y = (y & 0x83ff83ffu) | 0x38003800u; }  // binary16 in +-[0.5, 1)
    a[i][j] = (int)x; b[i][j] = (int)y;
  }
  int sink = 0;
  if (KIND == 0) {
    v16i acc[16]; for (auto &c : acc) c = v16i(0);
    for (int it = 0; it < iters; ++it)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[4 * i + j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i + 4 * (it & 1)], b[j + 4 * (it & 1)], acc[4 * i + j], 0, 0, 0);
    for (auto &c : acc) for (int e = 0; e < 16; ++e) sink ^= c[e];
  } else if (KIND == 1) {
    v4i acc[64]; for (auto &c : acc) c = v4i(0);
    for (int it = 0; it < iters; ++it)
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[8 * i + j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[i], b[j], acc[8 * i + j], 0, 0, 0);
    for (auto &c : acc) for (int e = 0; e < 4; ++e) sink ^= c[e];
  } else if (KIND == 2) {
    v16f acc[16]; for (auto &c : acc) c = v16f(0.f);
    for (int it = 0; it < iters; ++it)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc[4 * i + j]) : "v"(a[i + 4 * (it & 1)]), "v"(b[j + 4 * (it & 1)]));
    for (auto &c : acc) for (int e = 0; e < 16; ++e) sink ^= __builtin_bit_cast(int, c[e]);
  } else {
    v4f acc[64]; for (auto &c : acc) c = v4f(0.f);
    for (int it = 0; it < iters; ++it)
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j)
          asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[8 * i + j]) : "v"(a[i]), "v"(b[j]));
    for (auto &c : acc) for (int e = 0; e < 4; ++e) sink ^= __builtin_bit_cast(int, c[e]);
  }
  if (sink == 0x12345678) out[0] = sink;
}
static double board_power() {
  FILE *f = fopen("/sys/class/drm/card0/device/hwmon/hwmon0/power1_input", "r");
  if (!f) return -1;
  long long v = 0;
  if (fscanf(f, "%lld", &v) != 1) v = -1000000;
  fclose(f);
  return v / 1e6;
}
static int mfma_main() {
  int *out; CK(hipMalloc(&out, 64));
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  const char *names[4] = {"v_mfma_i32_32x32x32_i8", "v_mfma_i32_16x16x64_i8", "v_mfma_f32_32x32x16_f16", "v_mfma_f32_16x16x32_f16"};
  const double ops[4] = {16 * 65536.0, 64 * 32768.0, 16 * 32768.0, 64 * 16384.0};   // per wave and iteration
  for (int rep = 0; rep < 2; ++rep)
    for (int kind = 0; kind < 4; ++kind) {
      auto kern = kind == 0 ? k_mfma<0> : kind == 1 ? k_mfma<1> : kind == 2 ? k_mfma<2> : k_mfma<3>;
      const int iters = kind & 1 ? 2000 : 4000;   // about a millisecond per launch
      hipLaunchKernelGGL(kern, 256, 256, 0, 0, out, iters); CK(hipGetLastError()); CK(hipDeviceSynchronize());
      const auto t0 = std::chrono::steady_clock::now();
      auto since = [&]() { return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count(); };
      double psum = 0; int pn = 0, launches = 0; float ms_total = 0;
      while (since() < 2.0) {
        CK(hipEventRecord(e0));
        for (int i = 0; i < 20; ++i) hipLaunchKernelGGL(kern, 256, 256, 0, 0, out, iters);
        CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
        float ms; CK(hipEventElapsedTime(&ms, e0, e1));
        if (since() > 1.0) { ms_total += ms; launches += 20; psum += board_power(); ++pn; }
      }
      printf("%-26s %.3f ms per launch  %.2f POP/s or PFLOP/s  %.0f W\n", names[kind], ms_total / launches,
             ops[kind] * iters * 4 * 256 / (ms_total / launches) / 1e12, pn ? psum / pn : -1.0);
    }
  return 0;
}
'''


def source():
    clob = ",".join(f'"v{r}"' for r in range(4, 128)) + "," + ",".join(f'"s{r}"' for r in range(16, 32)) + ',"scc"'
    out = ["// written by cuasr_amd/issue_probe.py", "#include <hip/hip_runtime.h>", "#include <cstdio>", "#include <cstdlib>", "#include <cstring>", "#include <chrono>",
           '#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("HIP error %s at %d\\n", hipGetErrorString(e), __LINE__); exit(1);} } while (0)']
    ks = kernels()
    for name, (lines, _, _, _) in ks.items():
        body = "\\n".join(lines + ["s_waitcnt lgkmcnt(0)"])
        out.append(f'''__global__ __launch_bounds__(256) void k_{name}(unsigned long long *out, int iters) {{
  __shared__ float lds[9216];
  for (int i = threadIdx.x; i < 9216; i += 256) lds[i] = i;
  __syncthreads();
  const unsigned addr = (unsigned)(size_t)(__attribute__((address_space(3))) float *)&lds[0] + (threadIdx.x & 63) * 16;
  const unsigned long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {{
    asm volatile("{body}" :: "v"(addr) : {clob});
  }}
  const unsigned long long c1 = __builtin_readcyclecounter(), w1 = wall_clock64();
  if (threadIdx.x == 0) {{ out[2 * blockIdx.x] = c1 - c0; out[2 * blockIdx.x + 1] = w1 - w0; }}
}}''')
    out.append(MFMA_SECTION)
    out.append('''int main(int argc, char **argv) {
  setvbuf(stdout, NULL, _IONBF, 0);
  if (argc > 1 && !strcmp(argv[1], "mfma")) return mfma_main();
  hipDeviceProp_t prop; CK(hipGetDeviceProperties(&prop, 0));
  unsigned long long *out, *h = (unsigned long long *)malloc(16 * 8192);
  CK(hipMalloc(&out, 16 * 8192));
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  const int iters = argc > 1 ? atoi(argv[1]) : 20000;
  printf("%s, %d compute units; %d iterations per launch\\n", prop.name, prop.multiProcessorCount, iters);
  for (int bpc : {1, 2, 3, 4}) {
    const int blocks = prop.multiProcessorCount * bpc;
    auto run = [&](auto kern, const char *name, double ninstr, double terms, double ops_per_term) {
      hipLaunchKernelGGL(kern, blocks, 256, 0, 0, out, iters); CK(hipDeviceSynchronize());
      CK(hipEventRecord(e0)); hipLaunchKernelGGL(kern, blocks, 256, 0, 0, out, iters); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
      float ms; CK(hipEventElapsedTime(&ms, e0, e1));
      CK(hipMemcpy(h, out, 16 * blocks, hipMemcpyDeviceToHost));
      double cyc = 0, wall = 0; for (int b = 0; b < blocks; ++b) { cyc += h[2 * b]; wall += h[2 * b + 1]; }
      const double ghz = cyc / (wall * 10.0);   // the wall clock ticks at 100 MHz
      printf("waves/SIMD %d  %-22s %8.3f ms  %.2f GHz  %5.2f cycles per counted instruction and SIMD", bpc, name, ms, ghz,
             ms * 1e-3 * ghz * 1e9 / (ninstr * iters * bpc));
      if (terms > 0) printf("  %6.1f TOPS", ops_per_term * terms * iters * 256.0 * blocks / ms / 1e9);
      printf("\\n");
    };''')
    for name, (_, ninstr, terms, _) in ks.items():
        out.append(f'    run(k_{name}, "{name}", {ninstr}, {terms}, 2.0);')
    out.append("  }\n  return 0;\n}")
    return "\n".join(out)


def build():
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    src = os.path.join(HERE, "build", "issue_probe.hip")
    with open(src, "w") as f:
        f.write(source())
    subprocess.check_call([HIPCC, "--offload-arch=gfx950", "-O3", "-w", "-o", OUT, src])
    return OUT


if __name__ == "__main__":
    if "--build" in sys.argv:
        print(build())
    else:
        print(__doc__)
