/* Host check of the reciprocal refinement used by the single-precision sigmoid (cta_rcp_refined in
 * ctorch_amd/csrc/devmath.h): a starting value within 1 ulp of 1 / s (what the hardware reciprocal
 * returns), two Newton steps r <- r + r (1 - s r) with fused multiply-adds.  Every significand of
 * s in [1, 2) with the three starting values (correctly rounded, one below, one above); powers of
 * two scale exactly, so one binade covers all normal s.  Prints "tested N bad M allones K": M counts
 * results that are not the correctly rounded quotient for significands other than all ones, K the
 * (expected: 1 ulp low) results for the all-ones significand. */
#include <stdio.h>
#include <stdint.h>
#include <string.h>
#include <math.h>
static float u2f(uint32_t u){float f;memcpy(&f,&u,4);return f;}
static uint32_t f2u(float f){uint32_t u;memcpy(&u,&f,4);return u;}
int main(void){
  long bad=0,ones=0,n=0;
  for(uint32_t m=0;m<(1u<<23);++m){
    float s=u2f(0x3f800000u|m);
    float want=1.0f/s;
    for(int d=-1;d<=1;++d){
      float r=u2f(f2u(want)+(uint32_t)d);
      r=fmaf(fmaf(-s,r,1.0f),r,r);
      r=fmaf(fmaf(-s,r,1.0f),r,r);
      ++n;
      if(r!=want){
        if(m==(1u<<23)-1 && f2u(want)-f2u(r)==1u) ++ones; else ++bad;
      }
    }
  }
  printf("tested %ld bad %ld allones %ld\n",n,bad,ones);
  return 0;
}
