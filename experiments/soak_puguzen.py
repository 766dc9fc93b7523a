"""Randomised soak of the Puguzen family: random layer lists (mixer kinds, head counts, sizes that
divide nothing, rotary dims, windows, pools, ranks, with and without a feed-forward), three
requests of random lengths fed in random portions and mixed batches, float32 and bfloat16 engines
against the plain CPU model (oracle/puguzen.py).

    python experiments/soak_puguzen.py [seed] [configurations]
"""
import os
import random
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from oracle import puguzen as P
from vllm_omni_draft_amd import config, weights
from vllm_omni_draft_amd.seq_engine import SeqEngine, SeqEngineConfig
def rel(a,b):
    a,b=a.double().cpu(),b.double().cpu(); return ((a-b).pow(2).mean().sqrt()/b.pow(2).mean().sqrt()).item()
rng=random.Random(int(sys.argv[1]) if len(sys.argv)>1 else 0)
def rand_layer(W):
    kind=rng.choice(["retention","gla","attention"])
    H=rng.choice([1,2,3,4,6,8]); dk=rng.choice([8,16,24,32,40,48,64,96,128]); dv=rng.choice([8,16,24,32,48,64,72,128])
    m=dict(heads=H,dim=dk,vdim=dv)
    if kind=="retention":
        m["decay"]=[1-2.0**-(2+rng.random()*6) for _ in range(H)]
        m["rot"]={"dims":rng.choice([dk,dk//2-(dk//2)%2,2]),"base":rng.choice([100.0,1e4,1e6])}
    elif kind=="gla":
        m["tau"]=rng.choice([1.0,4.0,16.0,64.0]); m["rank"]=rng.choice([1,4,16,32,7])
    else:
        G=rng.choice([g for g in (1,2,3,4,6,8) if H%g==0]); m["kv_heads"]=G
        m["rot"]={"dims":rng.choice([dk,dk//2-(dk//2)%2,2]),"base":rng.choice([100.0,1e4,5e5])}
        m["scale"]=rng.choice([0.125,0.25,dk**-0.5,1.0]); m["mask"]={"size":rng.choice([1,3,16,17,40,100,64]),"pool":rng.choice([1,2,4,5,8,16,24,32])}
    ff=rng.choice([0,W,2*W,W+W//2,100,288])
    return {"type":kind,"mixer":m,"mlp":{"kind":"dense","ff":ff} if ff else None}
for it in range(int(sys.argv[2]) if len(sys.argv)>2 else 12):
    W=rng.choice([32,64,96,128,160,224,200,72]); V=rng.choice([64,130,256,500,1000])
    cfg={"architecture":"Puguzen","width":W,"vocab":V,"norm":{"eps":rng.choice([1e-5,1e-6])},"layers":[rand_layer(W) for _ in range(rng.choice([1,2,3,4,5]))]}
    st=P.random_model(cfg, it)
    mc=config.puguzen_config(cfg,{k:tuple(v.shape) for k,v in st.items()})
    desc=[(l["type"],l["mixer"]["heads"],l["mixer"].get("kv_heads"),l["mixer"]["dim"],l["mixer"]["vdim"],l["mixer"].get("mask"),l["mixer"].get("rot",{}).get("dims"),l["mixer"].get("rank"),(l["mlp"] or {}).get("ff")) for l in cfg["layers"]]
    print(it,"W",W,"V",V,desc,flush=True)
    lens=[rng.randint(1,300) for _ in range(3)]
    g=torch.Generator().manual_seed(it)
    toks=[torch.randint(0,V,(n,),generator=g).tolist() for n in lens]
    refs=[P.forward(cfg,st,t,P.Sequence(cfg)) for t in toks]
    for dt,tol in ((torch.float32,2e-5),(torch.bfloat16,0.05)):
        w=weights.seq_from_state_dict(mc,st,"cuda",dt)
        eng=SeqEngine(w,SeqEngineConfig(max_seqs=4,max_tokens=1024,max_seq_len=320,max_rows=rng.choice([64,2048])))
        at=[0,0,0]; got=[[],[],[]]
        while any(at[i]<lens[i] for i in range(3)):
            ents=[]
            for i in range(3):
                if at[i]<lens[i] and rng.random()<0.8:
                    c=min(lens[i]-at[i], rng.choice([1,1,1,2,3,17,64,130]))
                    ents.append((i,c))
            if not ents: continue
            out=eng.step([(f"r{i}",toks[i][at[i]:at[i]+c],list(range(c))) for i,c in ents]).cpu()
            o=0
            for i,c in ents:
                got[i].append(out[o:o+c]); o+=c; at[i]+=c
        worst=max(rel(torch.cat(got[i]),refs[i]) for i in range(3))
        print("   ",dt,"worst rel",worst, "replays",eng.graph_replays, flush=True)
        assert worst<tol,(it,dt,worst)
print("soak ok")
