

JP=ؐ===Wַ==d=Wַ=Wַ====M==ѷ=W=f=ѷ=ѷ=)=Boutput_0