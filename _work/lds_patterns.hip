// LDS access-pattern micro-benchmark for gfx950: cycles per wave-instruction of the access patterns the
// sweep kernels use (16-byte and 8-byte fragment reads, transpose reads, staging writes), by row stride
// and by the number of wavefronts on the CU.  One workgroup; every wavefront issues batches of eight
// independent accesses and waits once per batch, so the figures are throughput, not latency.
//
//     hipcc --offload-arch=gfx950 -O2 lightning-attention_amd/benchmarks/lds_patterns.hip -o /tmp/lds_patterns && /tmp/lds_patterns
//
// Columns: row stride in bytes (272 / 288 / 304 = 128 bf16 features + 8 / 16 / 24 of padding; 136 .. 176 the
// same for 64 features).  Rows: pattern x wavefronts.  "--": a 16-byte access needs 16-byte aligned rows.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
typedef __attribute__((__vector_size__(4 * sizeof(int)))) int i32x4;
typedef __attribute__((__vector_size__(2 * sizeof(int)))) int i32x2;
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("ERR %s: %s\n",#x,hipGetErrorString(e)); exit(1);} }while(0)
enum {B128, B64, TR64, W128, W64};
template<int KIND>
__global__ void k(int pattern, int stride_b, int iters, long long* out, int* sink){
  extern __shared__ __align__(16) unsigned char lds[];
  int l = threadIdx.x & 63;
  for(int i=threadIdx.x;i<65536/4;i+=blockDim.x) ((int*)lds)[i]=i;
  __syncthreads();
  unsigned off=0;
  int r16=l%16,g=l/16,r32=l%32,G=l/32,L=l%16;
  switch(pattern){
    case 0: off=r16*stride_b+16*g; break;            // b128 rows r16 chunk g
    case 1: off=r32*stride_b+16*G; break;            // b128 rows r32 chunk G
    case 2: off=r16*stride_b+8*g; break;             // b64 rows r16, 8B*g
    case 3: off=r32*stride_b+8*G; break;             // b64 rows r32
    case 4: off=(8*g+(L/4))*stride_b+8*(L%4); break; // tr16 natural
    case 5: off=(8*g+(L/4))*stride_b+16*(L%4); break;// tr16 perm (8-elem chunks)
    case 6: off=(l/16)*stride_b+16*(l%16); break;    // row-major staging 256B rows
    case 7: off=(l/8)*stride_b+16*(l%8); break;      // row-major staging 128B rows
    case 8: off=(8*G+(L/4))*stride_b+32*(g%2)+8*(L%4); break; // tr 32x32 pattern
  }
  unsigned addr = off + (threadIdx.x>>6)*0; // all waves same region
  i32x4 a0,a1,a2,a3,a4,a5,a6,a7; i32x2 b0,b1,b2,b3,b4,b5,b6,b7;
  i32x4 acc={0,0,0,0};
  a0=a1=a2=a3=a4=a5=a6=a7=acc; b0=b1=b2=b3=b4=b5=b6=b7=(i32x2){0,0};
  long long t0=clock64();
  for(int it=0;it<iters;it++){
    if(KIND==B128){
      asm volatile("ds_read_b128 %0, %8\n ds_read_b128 %1, %8 offset:4608\n ds_read_b128 %2, %8 offset:9216\n ds_read_b128 %3, %8 offset:13824\n"
                   "ds_read_b128 %4, %8 offset:18432\n ds_read_b128 %5, %8 offset:23040\n ds_read_b128 %6, %8 offset:27648\n ds_read_b128 %7, %8 offset:32256\n s_waitcnt lgkmcnt(0)"
        : "=v"(a0),"=v"(a1),"=v"(a2),"=v"(a3),"=v"(a4),"=v"(a5),"=v"(a6),"=v"(a7) : "v"(addr));
      acc += a0^a1^a2^a3^a4^a5^a6^a7;
    } else if(KIND==B64){
      asm volatile("ds_read_b64 %0, %8\n ds_read_b64 %1, %8 offset:4608\n ds_read_b64 %2, %8 offset:9216\n ds_read_b64 %3, %8 offset:13824\n"
                   "ds_read_b64 %4, %8 offset:18432\n ds_read_b64 %5, %8 offset:23040\n ds_read_b64 %6, %8 offset:27648\n ds_read_b64 %7, %8 offset:32256\n s_waitcnt lgkmcnt(0)"
        : "=v"(b0),"=v"(b1),"=v"(b2),"=v"(b3),"=v"(b4),"=v"(b5),"=v"(b6),"=v"(b7) : "v"(addr));
      i32x2 x=b0^b1^b2^b3^b4^b5^b6^b7; acc[0]+=x[0]; acc[1]+=x[1];
    } else if(KIND==TR64){
      asm volatile("ds_read_b64_tr_b16 %0, %8\n ds_read_b64_tr_b16 %1, %8 offset:4608\n ds_read_b64_tr_b16 %2, %8 offset:9216\n ds_read_b64_tr_b16 %3, %8 offset:13824\n"
                   "ds_read_b64_tr_b16 %4, %8 offset:18432\n ds_read_b64_tr_b16 %5, %8 offset:23040\n ds_read_b64_tr_b16 %6, %8 offset:27648\n ds_read_b64_tr_b16 %7, %8 offset:32256\n s_waitcnt lgkmcnt(0)"
        : "=v"(b0),"=v"(b1),"=v"(b2),"=v"(b3),"=v"(b4),"=v"(b5),"=v"(b6),"=v"(b7) : "v"(addr));
      i32x2 x=b0^b1^b2^b3^b4^b5^b6^b7; acc[0]+=x[0]; acc[1]+=x[1];
    } else if(KIND==W128){
      asm volatile("ds_write_b128 %0, %1\n ds_write_b128 %0, %1 offset:4608\n ds_write_b128 %0, %1 offset:9216\n ds_write_b128 %0, %1 offset:13824\n"
                   "ds_write_b128 %0, %1 offset:18432\n ds_write_b128 %0, %1 offset:23040\n ds_write_b128 %0, %1 offset:27648\n ds_write_b128 %0, %1 offset:32256\n s_waitcnt lgkmcnt(0)"
        :: "v"(addr),"v"(acc) : "memory");
    } else {
      i32x2 w={acc[0],acc[1]};
      asm volatile("ds_write_b64 %0, %1\n ds_write_b64 %0, %1 offset:4608\n ds_write_b64 %0, %1 offset:9216\n ds_write_b64 %0, %1 offset:13824\n"
                   "ds_write_b64 %0, %1 offset:18432\n ds_write_b64 %0, %1 offset:23040\n ds_write_b64 %0, %1 offset:27648\n ds_write_b64 %0, %1 offset:32256\n s_waitcnt lgkmcnt(0)"
        :: "v"(addr),"v"(w) : "memory");
    }
  }
  long long t1=clock64();
  if(threadIdx.x==0) out[blockIdx.x]=t1-t0;
  sink[threadIdx.x]=acc[0]+acc[1]+acc[2]+acc[3];
}
typedef void (*KF)(int,int,int,long long*,int*);
int main(){
  long long* d; int* s; CK(hipMalloc(&d,8*16)); CK(hipMalloc(&s,4*1024));
  struct Case{const char* name; int kind; int pattern;};
  Case cases[]={{"b128 r16/g",B128,0},{"b128 r32/G",B128,1},{"b64 r16/g",B64,2},{"b64 r32/G",B64,3},{"tr16 nat",TR64,4},{"tr16 perm",TR64,5},{"tr32",TR64,8},
                {"w128 r16/g",W128,0},{"w128 rowmaj256",W128,6},{"w128 rowmaj128",W128,7},{"w64 r16/g",W64,2}};
  KF fs[]={k<B128>,k<B64>,k<TR64>,k<W128>,k<W64>};
  for(auto f:fs) CK(hipFuncSetAttribute((const void*)f, hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
  int strides[]={264,272,280,288,304,136,144,152,160,176};
  int iters=2000;
  printf("cycles per wave-instruction aggregated over the CU (elapsed / (iters*8*waves))\n%-16s waves","case");
  for(int st:strides) printf(" %6d",st); printf("\n");
  for(auto& c:cases) for(int waves : {1,4,8,16}){
    printf("%-16s %5d",c.name,waves);
    for(int st:strides){
      if((c.kind==B128||c.kind==W128)&&(st%16)) { printf("     --"); continue; }
      fs[c.kind]<<<1,64*waves,65536>>>(c.pattern,st,iters,d,s); CK(hipDeviceSynchronize());
      long long h; CK(hipMemcpy(&h,d,8,hipMemcpyDeviceToHost));
      printf(" %6.2f",(double)h/(iters*8.0*waves));
    }
    printf("\n");
  }
  return 0;
}
