// Measures the hardware ceilings the GEMM kernels are judged against on one MI355X (gfx950), each with the core
// clock it sustains (core cycles / 100 MHz wall ticks):
//   LDS read bandwidth (ds_read_b128: contiguous and the tiled kernel's swizzled A-fragment pattern),
//   MFMA-only rates (fp8 16x16x128, int8 16x16x64, fp4 16x16x128 scaled) on random and on zero operands, with one
//   and with two wavefronts per SIMD, L2-hit vector load bandwidth per CU, HBM write bandwidth,
//   a plain read of a decode-sized weight (25.2 MB) rotating through 25 copies and from the Infinity Cache,
//   the launch floor of an empty kernel, and the small-M streaming GEMM (fp8, M=16, N=6144, K=4096) as the library
//   launches it, with its parts switched off one at a time (what A, the in-workgroup reduction and the store cost).
// Build: make -C flydsl_amd/csrc ../psg_ceilings      Run: flydsl_amd/psg_ceilings
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <vector>
#include "gemm_a8w8_stream.hip"  // the library's small-M kernel (and the vector typedefs of psg_common.h)
typedef float v16f __attribute__((ext_vector_type(16)));
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("HIP error %s at %d\n",hipGetErrorString(e),__LINE__); exit(1);} }while(0)

// ---- LDS read bandwidth: every wavefront of every CU reads its own 8 KB window, 8 independent reads in flight ----
// PAT 0: lane l reads 16 bytes at l*16 (+1 KB per read): contiguous.  PAT 1: the A-fragment pattern of the tiled
// kernel: lane (i = l%16, g = l/16) reads row i (128-byte rows, XOR swizzle of the 16-byte chunk by (i/2)%8).
template<int PAT>
__global__ void __launch_bounds__(512) k_lds(int iters, unsigned long long* out){
  __shared__ __attribute__((aligned(16))) char lds[65536];
  for(int i=threadIdx.x;i<16384;i+=blockDim.x) ((int*)lds)[i]=i;
  __syncthreads();
  int lane=threadIdx.x&63, wave=threadIdx.x>>6;
  unsigned off = PAT==0 ? lane*16 : ((lane&15)*128 + (((lane>>4) ^ (((lane&15)>>1)&7))<<4));
  unsigned addr = (unsigned)(size_t)(lds) + wave*8192 + off;
  v4i a0,a1,a2,a3,a4,a5,a6,a7; v4i acc={0,0,0,0};
  unsigned long long w0=wall_clock64(); long long t0=clock64();
  for(int it=0;it<iters;it++){
    if(PAT==0)
    asm volatile("ds_read_b128 %0, %8\n ds_read_b128 %1, %8 offset:1024\n ds_read_b128 %2, %8 offset:2048\n ds_read_b128 %3, %8 offset:3072\n"
                 "ds_read_b128 %4, %8 offset:4096\n ds_read_b128 %5, %8 offset:5120\n ds_read_b128 %6, %8 offset:6144\n ds_read_b128 %7, %8 offset:7168\n s_waitcnt lgkmcnt(0)"
                 : "=v"(a0),"=v"(a1),"=v"(a2),"=v"(a3),"=v"(a4),"=v"(a5),"=v"(a6),"=v"(a7) : "v"(addr) : "memory");
    else
    asm volatile("ds_read_b128 %0, %8\n ds_read_b128 %1, %8 offset:64\n ds_read_b128 %2, %8 offset:2048\n ds_read_b128 %3, %8 offset:2112\n"
                 "ds_read_b128 %4, %8 offset:4096\n ds_read_b128 %5, %8 offset:4160\n ds_read_b128 %6, %8 offset:6144\n ds_read_b128 %7, %8 offset:6208\n s_waitcnt lgkmcnt(0)"
                 : "=v"(a0),"=v"(a1),"=v"(a2),"=v"(a3),"=v"(a4),"=v"(a5),"=v"(a6),"=v"(a7) : "v"(addr) : "memory");
    acc ^= a0^a1^a2^a3^a4^a5^a6^a7;
  }
  long long t1=clock64(); unsigned long long w1=wall_clock64();
  if(lane==0){ out[(blockIdx.x*8+wave)*2]=t1-t0; out[(blockIdx.x*8+wave)*2+1]=w1-w0; }
  if(acc[0]+acc[1]+acc[2]+acc[3]==12345) out[0]=1;
}
// ---- MFMA only: 8 independent accumulators per wavefront, operands random or zero ----
// KIND 0: fp8 16x16x128 (65536 flop), 1: int8 16x16x64 (32768 op), 2: fp4 16x16x128 with e8m0 scales (65536 flop),
// 3: fp8 32x32x64 (131072 flop, four accumulators of 16 registers)
template<int KIND>
__global__ void __launch_bounds__(512) k_mfma(int iters, const int* src, unsigned long long* out){
  v8i a, b; for(int i=0;i<8;i++){ a[i]=src[(threadIdx.x*8+i)&4095]; b[i]=src[(threadIdx.x*8+i+2048)&4095]; }
  v4i a4={a[0],a[1],a[2],a[3]}, b4={b[0],b[1],b[2],b[3]};
  v4f c[8]; v4i ci[8]; for(int i=0;i<8;i++){ c[i]=(v4f){0,0,0,0}; ci[i]=(v4i){0,0,0,0}; }
  v16f cw[4]; for(int i=0;i<4;i++) for(int j=0;j<16;j++) cw[i][j]=0.f;
  unsigned long long w0=wall_clock64(); long long t0=clock64();
  for(int it=0;it<iters;it++){
#pragma unroll
    for(int i=0;i<8;i++){
      if constexpr (KIND==3) cw[i&3]=__builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a,b,cw[i&3],0,0,0,0,0,0);
      else if constexpr (KIND==0) c[i]=__builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a,b,c[i],0,0,0,0,0,0);
      else if constexpr (KIND==1) ci[i]=__builtin_amdgcn_mfma_i32_16x16x64_i8(a4,b4,ci[i],0,0,0);
      else c[i]=__builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a,b,c[i],4,4,0,0x7f7f7f7f,0,0x7f7f7f7f);
    }
  }
  long long t1=clock64(); unsigned long long w1=wall_clock64();
  float s=0; for(int i=0;i<8;i++) s+=c[i][0]+(float)ci[i][0]+cw[i&3][i];
  if((threadIdx.x&63)==0){ int w=blockIdx.x*(blockDim.x/64)+(threadIdx.x>>6); out[w*2]=t1-t0; out[w*2+1]=w1-w0; }
  if(s==12345.f) out[0]=1;
}
// ---- L2-hit vector loads: every wavefront re-reads the same 64 KB with 16-byte loads ----
__global__ void __launch_bounds__(256) k_l2(int iters, const v4i* src, unsigned long long* out){
  int lane=threadIdx.x&63, wave=threadIdx.x>>6; const v4i* p=src+(blockIdx.x%64)*4096+wave*1024+lane;
  v4i acc={0,0,0,0};
  unsigned long long w0=wall_clock64(); long long t0=clock64();
  for(int it=0;it<iters;it++){
    v4i v[8];
#pragma unroll
    for(int i=0;i<8;i++) v[i]=__builtin_nontemporal_load(p+((i*64+it*512)&1023)*1+0);
#pragma unroll
    for(int i=0;i<8;i++) acc^=v[i];
  }
  long long t1=clock64(); unsigned long long w1=wall_clock64();
  if(lane==0){ int w=blockIdx.x*4+wave; out[w*2]=t1-t0; out[w*2+1]=w1-w0; }
  if(acc[0]+acc[1]+acc[2]+acc[3]==12345) out[0]=1;
}
__global__ void k_empty(){}
__global__ void __launch_bounds__(256) k_write(v4i* dst){
  size_t i=((size_t)blockIdx.x*256+threadIdx.x); v4i v={(int)i,1,2,3};
#pragma unroll
  for(int k=0;k<8;k++) dst[i+(size_t)k*gridDim.x*256]=v;
}
template<int PER>
__global__ void __launch_bounds__(256) k_read(const v4i* b, int nwaves, int* out){
  int wave=blockIdx.x*4+(threadIdx.x>>6), lane=threadIdx.x&63; if(wave>=nwaves) return;
  const v4i* q=b+(size_t)wave*PER*64+lane; v4i v[PER];
#pragma unroll
  for(int i=0;i<PER;i++) v[i]=__builtin_nontemporal_load(q+i*64);
  v4i acc={0,0,0,0};
#pragma unroll
  for(int i=0;i<PER;i++) acc^=v[i];
  if(acc[0]+acc[1]+acc[2]+acc[3]==0x12345) out[0]=1;
}
int main(){
  unsigned long long* d; size_t n=256*16*2; CK(hipMalloc(&d,n*8)); std::vector<unsigned long long> h(n);
  auto report=[&](const char* name, int waves_total, double bytes_or_flop_per_wave, const char* unit, double scale){
    CK(hipDeviceSynchronize()); CK(hipMemcpy(h.data(),d,n*8,hipMemcpyDeviceToHost));
    double clk=0, wall=0; for(int w=0;w<waves_total;w++){ clk+=h[w*2]; wall+=h[w*2+1]; } clk/=waves_total; wall/=waves_total;
    double mhz = clk/(wall*0.01); // wall ticks are 10 ns
    printf("%-58s %8.1f %s per clk per CU   clock %.0f MHz   %.1f %s\n", name, bytes_or_flop_per_wave*(waves_total/256.0)/clk, unit, mhz, bytes_or_flop_per_wave*waves_total/(wall*1e-8)/scale, unit[0]=='B'?"TB/s chip":"TFLOP/s chip");
  };
  int iters=4000;
  for(int th: {256,512}){ char nm[96];
    k_lds<0><<<256,th>>>(iters,d); snprintf(nm,96,"LDS ds_read_b128 contiguous, %d waves/CU",th/64); report(nm,256*th/64,(double)iters*8*1024,"B",1e12);
    k_lds<1><<<256,th>>>(iters,d); snprintf(nm,96,"LDS ds_read_b128 A-fragment pattern, %d waves/CU",th/64); report(nm,256*th/64,(double)iters*8*1024,"B",1e12);
  }
  int* src; CK(hipMalloc(&src,4096*4)); std::vector<int> hs(4096);
  // operand data: "random" = random bytes with the top bit of every nibble clear (all fp8 values positive), "zero",
  // "signed" = fp8 bytes with random sign, exponent field 4..10 and random mantissa (what quantised GEMM operands look like)
  for(int mode=0;mode<3;mode++){
    for(auto&x:hs){ if(mode==0) x=rand()&0x77777777; else if(mode==1) x=0; else { unsigned v=0; for(int b=0;b<4;b++) v|=(unsigned)(((rand()&1)<<7)|(((rand()%7)+4)<<3)|(rand()&7))<<(8*b); x=(int)v; } }
    CK(hipMemcpy(src,hs.data(),4096*4,hipMemcpyHostToDevice));
    const char* dn = mode==0 ? "random" : (mode==1 ? "zero" : "signed");
    for(int th: {256,512}){ char nm[96]; int w=256*th/64;
      k_mfma<0><<<256,th>>>(100000,src,d); snprintf(nm,96,"MFMA only fp8 16x16x128, %s operands, %d waves/SIMD",dn,th/256); report(nm,w,(double)100000*8*65536,"flop",1e12);
      k_mfma<1><<<256,th>>>(200000,src,d); snprintf(nm,96,"MFMA only int8 16x16x64, %s operands, %d waves/SIMD",dn,th/256); report(nm,w,(double)200000*8*32768,"flop",1e12);
      k_mfma<2><<<256,th>>>(200000,src,d); snprintf(nm,96,"MFMA only fp4 16x16x128 scaled, %s operands, %d waves/SIMD",dn,th/256); report(nm,w,(double)200000*8*65536,"flop",1e12);
      k_mfma<3><<<256,th>>>(50000,src,d); snprintf(nm,96,"MFMA only fp8 32x32x64, %s operands, %d waves/SIMD",dn,th/256); report(nm,w,(double)50000*8*131072,"flop",1e12);
    } }
  v4i* big; CK(hipMalloc(&big,(size_t)64*4096*16)); CK(hipMemset(big,1,(size_t)64*4096*16));
  k_l2<<<256,256>>>(4000,big,d); report("vector loads 16 B/lane hitting L2 (4 MB footprint), 4 waves/CU",1024,(double)4000*8*1024,"B",1e12);
  k_l2<<<512,256>>>(4000,big,d); report("same, 8 waves/CU",2048,(double)4000*8*1024,"B",1e12);
  { // HBM write bandwidth: 1 GiB of 16-byte stores
    size_t wb=(size_t)1<<30; v4i* wbuf; CK(hipMalloc(&wbuf,wb)); hipEvent_t e0,e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1)); float best=1e9;
    for(int r=0;r<4;r++){ CK(hipEventRecord(e0)); k_write<<<(unsigned)(wb/16/256/8),256>>>(wbuf); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1)); float ms; CK(hipEventElapsedTime(&ms,e0,e1)); if(ms<best)best=ms; }
    printf("%-58s %.1f us for 1 GiB  %.0f GB/s\n","plain write, 16-byte stores",best*1e3,wb/(best*1e-3)/1e9); CK(hipFree(wbuf)); }
  // rotating plain read + empty kernel, graph-timed
  size_t bbytes=(size_t)6144*4096; int sets=25; std::vector<v4i*> bs(sets); for(auto&p:bs){ CK(hipMalloc(&p,bbytes)); CK(hipMemset(p,0x11,bbytes)); }
  int* dout; CK(hipMalloc(&dout,4)); hipStream_t st; CK(hipStreamCreate(&st)); int steps=400;
  auto run=[&](const char* name, auto launch){
    hipGraph_t g; hipGraphExec_t ge; CK(hipStreamBeginCapture(st,hipStreamCaptureModeGlobal)); for(int i=0;i<steps;i++) launch(i%sets);
    CK(hipStreamEndCapture(st,&g)); CK(hipGraphInstantiate(&ge,g,nullptr,nullptr,0)); CK(hipGraphLaunch(ge,st)); CK(hipStreamSynchronize(st));
    hipEvent_t e0,e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1)); float best=1e9;
    for(int r=0;r<4;r++){ CK(hipEventRecord(e0,st)); CK(hipGraphLaunch(ge,st)); CK(hipEventRecord(e1,st)); CK(hipEventSynchronize(e1)); float ms; CK(hipEventElapsedTime(&ms,e0,e1)); if(ms<best)best=ms; }
    printf("%-58s %.2f us per launch (graph of %d)  %.0f GB/s\n",name,best*1e3/steps,steps,bbytes/(best*1e-3/steps)/1e9); };
  run("plain read of 25.2 MB, rotating 25 sets, 24 KB per wave", [&](int i){ int nw=bbytes/(24*1024); k_read<24><<<(nw+3)/4,256,0,st>>>(bs[i],nw,dout); });
  run("plain read of 25.2 MB, rotating 25 sets, 12 KB per wave", [&](int i){ int nw=bbytes/(12*1024); k_read<12><<<(nw+3)/4,256,0,st>>>(bs[i],nw,dout); });
  run("plain read of 25.2 MB, one set (Infinity Cache hot)", [&](int i){ int nw=bbytes/(24*1024); k_read<24><<<(nw+3)/4,256,0,st>>>(bs[0],nw,dout); });
  run("empty kernel, 256 x 512 threads", [&](int i){ k_empty<<<256,512,0,st>>>(); });
  { // the streaming GEMM of the decode shape, launched like the library does (256 workgroups x 8 wavefronts, 8 K slices,
    // 768 eight-column units dealt out 3 per workgroup, chunks of 2 K steps); A, scales and C stay fixed, W rotates
    const int M=16,N=6144,K=4096; uint8_t* a; float *sa,*sb; uint16_t* c;
    CK(hipMalloc(&a,(size_t)32*K)); CK(hipMemset(a,0x38,(size_t)32*K)); CK(hipMalloc(&sa,4*32)); CK(hipMalloc(&sb,4*N)); CK(hipMemset(sa,0,4*32)); CK(hipMemset(sb,0,4*N)); CK(hipMalloc(&c,(size_t)32*N*2));
    A8W8Params p{}; p.c=c; p.a=a; p.sa=sa; p.sb=sb; p.M=M; p.N=N; p.K=K; p.epi=EPI_NONE; p.out=OUT_BF16; p.ksplit=8; p.splits=256; p.group_m=(N/8)/256; p.wave_layout=(N/8)%256;
#define GEMM_DIAG(D,TXT) run(TXT, [&](int i){ A8W8Params q=p; q.b=(const uint8_t*)bs[i]; hipLaunchKernelGGL((k_a8w8_stream<KIND_FP8,1,2,8,2,STORE_C,D>),dim3(256),dim3(512),0,st,q); });
    GEMM_DIAG(0,"fp8 GEMM M=16 6144x4096, streaming kernel as shipped")
    GEMM_DIAG(1,"  same, A loads redirected past the bound")
    GEMM_DIAG(2,"  same, wavefronts end after their MFMAs")
    GEMM_DIAG(3,"  same, neither A nor reduction / store")
    GEMM_DIAG(4,"  same, reduction kept, nothing stored")
  }
  return 0;
}
