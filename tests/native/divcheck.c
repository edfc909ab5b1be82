/* Host check of cta_div_rcp (ctorch_amd/csrc/devmath.h): division by a shared divisor through its
 * double-precision reciprocal against IEEE fp32 division, on random operand pairs that include
 * subnormal numerators and divisors, numerators <= 1 with divisors >= 1 (the softmax case) and the
 * full exponent range, then on the family whose exact quotient is a midpoint between two subnormal
 * floats (a = M * B * 2^-149 with M odd, b = 2 * B: the quotient is (M / 2) * 2^-149), both signs.
 * Usage: divcheck [PAIRS_PER_THREAD]; prints "tested N bad M" and "ties N bad M". */
#include <stdio.h>
#include <stdint.h>
#include <string.h>
#include <math.h>
#include <stdlib.h>
#include "../../ctorch_amd/csrc/devmath.h"
static float u2f(uint32_t u){float f;memcpy(&f,&u,4);return f;}
static uint32_t f2u(float f){uint32_t u;memcpy(&u,&f,4);return u;}
static uint64_t rng(uint64_t*s){*s^=*s<<13;*s^=*s>>7;*s^=*s<<17;return *s;}
int main(int argc,char**argv){
  long per=argc>1?atol(argv[1]):40000000L;
  uint64_t bad=0,total=0;
  #pragma omp parallel for reduction(+:bad,total)
  for(int t=0;t<64;++t){
    uint64_t s=0x9E3779B97F4A7C15ULL*(t+1);
    for(long i=0;i<per;++i){
      uint32_t ua=(uint32_t)rng(&s), ub=(uint32_t)rng(&s);
      int mode=i%4;
      if(mode==1){ ua=(ua&0x807fffffu)|((uint32_t)(rng(&s)%40)<<23); }           /* tiny / subnormal numerators */
      if(mode==2){ ub=(ub&0x807fffffu)|((uint32_t)(127+rng(&s)%32)<<23); ua=(ua&0x807fffffu)|((uint32_t)(rng(&s)%128)<<23);} /* s>=1, e<=1 */
      if(mode==3){ ub=(ub&0x807fffffu)|((uint32_t)(rng(&s)%3)<<23); }              /* subnormal / tiny divisors */
      float a=u2f(ua), b=u2f(ub);
      volatile double rb=1.0/(double)b;
      float q1=cta_div_rcp(a,rb);
      float q2=a/b;
      ++total;
      if(!((q1!=q1)&&(q2!=q2)) && f2u(q1)!=f2u(q2)){ ++bad; if(bad<5) printf("a=%a b=%a fast=%a ieee=%a\n",a,b,q1,q2);}
    }
  }
  printf("tested %llu bad %llu\n",(unsigned long long)total,(unsigned long long)bad);
  uint64_t tbad=0,ties=0;
  #pragma omp parallel for reduction(+:tbad,ties) schedule(dynamic,8)
  for(int B=1;B<1024;++B){
    for(uint32_t M=1;(uint64_t)M*B<(1u<<24);M+=2){
      float a=ldexpf((float)(M*(uint32_t)B),-149), b=(float)(2*B);
      if(M&2){ a=-a; }
      volatile double rb=1.0/(double)b;
      float q1=cta_div_rcp(a,rb), q2=a/b;
      ++ties;
      if(f2u(q1)!=f2u(q2)){ ++tbad; if(tbad<5) printf("tie a=%a b=%a fast=%a ieee=%a\n",a,b,q1,q2);}
    }
  }
  printf("ties %llu bad %llu\n",(unsigned long long)ties,(unsigned long long)tbad);
  return 0;
}
