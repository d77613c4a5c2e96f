// Exhaustive check of the packed fp16 quantizer arithmetic (kvcomp_amd/csrc/kvc_quant_math.h, kvc_quant_pair_biased):
// for every finite fp16 x and every positive finite fp16 scale s with |x / s| <= 512, with P the power of two that
// brings s into [1, 2) (capped at 2^15), S = s * P, r = RN16(1 / S), X = RN16(x * P),
//   q0 = RN16(X * r),  rem = fma16(-q0, S, X),  q = fma16(rem, r, q0)
// must satisfy rint(q) == rint(RN16(x / s)) (the sign of a zero aside): the quantizer's symbol is that integer minus
// the group minimum.  All fp16 operations are modelled exactly (products and sums in 128-bit integers, one rounding
// to nearest even, subnormals kept).  argv[1] = "all": every scale; otherwise the scales of a spread of exponents
// (every mantissa of each).  Prints the pair count and the mismatch count.  Built and run by tests/test_fast_division.py.
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#include <omp.h>
typedef __int128 i128;
typedef struct { int neg; int64_t m; int e; int cls; } H;   // cls 0 finite, 1 inf, 2 nan
static H dec(uint16_t h){ H r; r.neg=h>>15; int ex=(h>>10)&31; int m=h&1023; r.cls=0; if(ex==31){ r.cls = m?2:1; r.m=0; r.e=0; return r;} if(ex==0){ r.m=m; r.e=-24; } else { r.m=m|1024; r.e=ex-25; } return r; }
static uint16_t rnd(int neg, i128 I, int E){   // I >= 0
  if(I==0) return (uint16_t)(neg<<15);
  int p=0; { i128 t=I; while(t>>1){ t>>=1; p++; } }
  int shift = p-10; if(shift < -24-E) shift = -24-E;
  i128 m; int e=E+shift;
  if(shift<=0) m = I << (-shift);
  else { i128 q=I>>shift, rem=I-(q<<shift), half=(i128)1<<(shift-1); if(rem>half || (rem==half && (q&1))) q++; m=q; }
  if(m>=2048){ m>>=1; e++; }     // only when m == 2048
  // now value = m * 2^e, m < 2048; normal iff m >= 1024
  if(m>=1024){ int ex=e+25; if(ex>=31) return (uint16_t)((neg<<15)|0x7c00); return (uint16_t)((neg<<15)|(ex<<10)|((int)m&1023)); }
  // subnormal: e must be -24
  return (uint16_t)((neg<<15)|(int)m);
}
static uint16_t fma16(uint16_t a, uint16_t b, uint16_t c){
  H x=dec(a), y=dec(b), z=dec(c);
  if(x.cls==2||y.cls==2||z.cls==2) return 0x7e00;
  if(x.cls==1||y.cls==1){ if((x.cls==0&&x.m==0)||(y.cls==0&&y.m==0)) return 0x7e00; int ns=x.neg^y.neg; if(z.cls==1 && z.neg!=ns) return 0x7e00; return (uint16_t)((ns<<15)|0x7c00); }
  if(z.cls==1) return c;
  int ep=x.e+y.e; i128 P=(i128)x.m*y.m; if(x.neg^y.neg) P=-P; i128 C=z.m; if(z.neg) C=-C;
  int E = ep<z.e?ep:z.e; i128 T=(P<<(ep-E))+(C<<(z.e-E));
  if(T==0){ int ns = ((x.neg^y.neg)&&z.neg); return (uint16_t)(ns<<15); }
  if(T<0) return rnd(1,-T,E); return rnd(0,T,E);
}
static uint16_t mul16(uint16_t a, uint16_t b){ return fma16(a,b,(uint16_t)(((a^b)&0x8000))); }
static double h2d(uint16_t h){ H x=dec(h); double v=ldexp((double)x.m,x.e); return x.neg?-v:v; }
static uint16_t d2h(double d){ // RNE double -> half, via exact integer (double has 53 bits)
  if(d==0) return signbit(d)?0x8000:0; int neg=d<0; if(neg)d=-d; if(isinf(d)) return (neg<<15)|0x7c00; int ex; double f=frexp(d,&ex); // d=f*2^ex, f in [.5,1)
  i128 I=(i128)ldexp(f,53); return rnd(neg,I,ex-53); }

static uint16_t rint16(uint16_t h){ double d=h2d(h); return d2h(nearbyint(d)); }
static uint16_t pow2h(int a){ return d2h(ldexp(1.0,a)); }
int main(int argc,char**argv){
  const int all = argc>1 && !strcmp(argv[1],"all");
  static const int quick[] = {0,1,2,9,13,14,15,16,17,21,29,30};
  long tot=0,bad=0,scales=0;
  #pragma omp parallel for reduction(+:tot,bad,scales) schedule(dynamic,64)
  for(int si=1; si<0x7c00; si++){
    int use=all; for(unsigned k=0;k<sizeof quick/sizeof quick[0];k++) if(((si>>10)&31)==quick[k]) use=1;
    if(!use) continue;
    scales++;
    uint16_t s=(uint16_t)si; double sd=h2d(s);
    int ex; frexp(sd,&ex); int a=1-ex; if(a>15) a=15;
    uint16_t P=pow2h(a), S=mul16(s,P); double Sd=h2d(S);
    if(Sd!=ldexp(sd,a)) { bad++; continue; }          // the scaled scale must be exact
    uint16_t r=d2h(1.0/Sd);
    for(int xi=0; xi<0x10000; xi++){
      if(((xi>>10)&31)==31) continue;
      uint16_t x=(uint16_t)xi; double q=h2d(x)/sd;
      if(fabs(q)>512.0) continue;
      uint16_t refi=rint16(d2h(q));
      uint16_t X=mul16(x,P), q0=mul16(X,r), rem=fma16(q0^0x8000,S,X), qf=fma16(rem,r,q0), qi=rint16(qf);
      tot++;
      if(qi!=refi && !((qi|refi)==0x8000)) bad++;
    }
  }
  printf("scales %ld pairs %ld mismatches %ld\n",scales,tot,bad);
  return 0;
}
