// Exhaustive check of the quantizer's three-instruction division (kvcomp_amd/csrc/kvc_quant_math.h,
// kvc_div_by_scale): for every finite fp16 x and every positive finite fp16 s, in fp32,
//   q_fast = fma(fma(-q0, s, x), r, q0),  q0 = RN(x * r),  r = RN(1 / s)
// must equal the IEEE quotient RN(x / s) bit for bit (the sign of a zero quotient aside), and
// RN16(q_fast) must equal RN16(RN(x / s)).  Prints the pair count and the two mismatch counts;
// mismatches whose quotient is a zero are counted separately.  Built and run by tests/test_fast_division.py.
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>
#include <omp.h>
static float h2f(uint16_t h){ uint32_t s=(h>>15)&1,e=(h>>10)&31,m=h&1023,u; if(e==0){ if(m==0){u=s<<31;} else { int k=0; while(!(m&1024)){m<<=1;k++;} m&=1023; u=(s<<31)|((uint32_t)(127-15-k+1)<<23)|(m<<13);} } else if(e==31){u=(s<<31)|0x7f800000u|(m<<13);} else u=(s<<31)|((e+112)<<23)|(m<<13); float f; memcpy(&f,&u,4); return f; }
#include <immintrin.h>
static uint16_t f2h(float f){ return (uint16_t)_cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT); }
int main(){
  long bad32=0,bad16=0,tot=0,zero=0;
  #pragma omp parallel for reduction(+:bad32,bad16,tot,zero) schedule(dynamic,64)
  for(int si=1; si<0x7c00; si++){
    float s=h2f((uint16_t)si); float r=1.0f/s;
    for(int xi=0; xi<0x10000; xi++){
      if(((xi>>10)&31)==31) continue;
      float x=h2f((uint16_t)xi);
      float q=x/s;
      float q0=x*r; float rem=fmaf(-q0,s,x); float qf=fmaf(rem,r,q0);
      uint32_t a,b; memcpy(&a,&q,4); memcpy(&b,&qf,4);
      tot++;
      if(a!=b){ if(q==0.0f && qf==0.0f) zero++; else { bad32++; if(f2h(q)!=f2h(qf)) bad16++; } }
    }
  }
  printf("pairs %ld fp32_mismatches %ld fp16_mismatches %ld zero_sign_only %ld\n",tot,bad32,bad16,zero);
  return 0;
}
